// Implementation of the Frame_HIP host cells and of their registrations.
#include "frame_hip.hpp"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <functional>
#include <cstring>

namespace N2D2 {

void checkStatus(int status)
{
    if (status != N2D2HIP_OK) {
        const char* msg = n2d2hip_last_error();
        throw std::runtime_error((msg && *msg) ? std::string(msg) : std::string(n2d2hip_strerror(status)));
    }
}

static void checkHip(hipError_t e, const char* what)
{
    if (e != hipSuccess)
        throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

// ------------------------------------------------------------------ HipTensor
HipTensor::~HipTensor()
{
    if (mDesc.data)
        (void)hipFree(mDesc.data);
}

void HipTensor::resize(int B, int C, int H, int W, int dtype, int halo, bool stimuli)
{
    n2d2hip_tensor d = {};
    d.data = nullptr;
    d.halo = halo;
    d.dtype = dtype;
    d.layout = N2D2HIP_NHWC;
    d.B = B; d.C = C; d.H = H; d.W = W;
    (void)stimuli;
    d.cs = n2d2hip_nhwc_cs(C);      // 4 for at most 4 channels (stimuli and cells alike), a multiple of 16 otherwise
    const size_t bytes = n2d2hip_tensor_bytes(&d);
    if (mDesc.data && bytes == mBytes) {
        d.data = mDesc.data;
    } else {
        if (mDesc.data)
            (void)hipFree(mDesc.data);
        mDesc.data = nullptr;
        checkHip(hipMalloc(&d.data, bytes), "HipTensor::resize(): hipMalloc");
        mBytes = bytes;
    }
    mDesc = d;
    mHostValid = false;
    if (halo > 0) {
        checkStatus(n2d2hip_tensor_clear(&mDesc, nullptr));
        checkHip(hipStreamSynchronize(nullptr), "HipTensor::resize(): clearing the halo");
    }
}

void HipTensor::resizeSpaceToDepth(int B, int C, int H, int W, int dtype, int halo)
{
    n2d2hip_tensor d = {};
    d.halo = halo;
    d.dtype = dtype;
    d.layout = N2D2HIP_S2D;
    d.B = B; d.C = C; d.H = H; d.W = W;
    d.cs = 16;
    const size_t bytes = n2d2hip_tensor_bytes(&d);
    if (mDesc.data && bytes == mBytes) {
        d.data = mDesc.data;
    } else {
        if (mDesc.data)
            (void)hipFree(mDesc.data);
        mDesc.data = nullptr;
        checkHip(hipMalloc(&d.data, bytes), "HipTensor::resizeSpaceToDepth(): hipMalloc");
        mBytes = bytes;
    }
    mDesc = d;
    mHostValid = false;
}

const Tensor<Float_T>& HipTensor::synchronizeDToH(void* stream)
{
    if (mHostValid)
        return mHost;
    if (!mDesc.data)
        throw std::runtime_error("HipTensor::synchronizeDToH(): empty tensor");
    n2d2hip_tensor f = mDesc;
    f.dtype = N2D2HIP_F32;
    f.layout = N2D2HIP_NCHW;
    f.halo = 0;
    const size_t n = (size_t)f.B * f.C * f.H * f.W;
    checkHip(hipMalloc(&f.data, n * sizeof(float)), "HipTensor::synchronizeDToH(): hipMalloc");
    int rc = n2d2hip_convert(&mDesc, &f, stream);
    mHost.resize({(size_t)f.W, (size_t)f.H, (size_t)f.C, (size_t)f.B});
    hipError_t e = hipSuccess;
    if (rc == N2D2HIP_OK) {
        e = hipStreamSynchronize((hipStream_t)stream);
        if (e == hipSuccess)
            e = hipMemcpy(mHost.data(), f.data, n * sizeof(float), hipMemcpyDeviceToHost);
    }
    (void)hipFree(f.data);
    checkStatus(rc);
    checkHip(e, "HipTensor::synchronizeDToH()");
    mHostValid = true;
    return mHost;
}

void HipTensor::synchronizeHToD(const Tensor<Float_T>& host, void* stream)
{
    if (!mDesc.data)
        throw std::runtime_error("HipTensor::synchronizeHToD(): empty tensor");
    if (host.dimX() != (size_t)mDesc.W || host.dimY() != (size_t)mDesc.H || host.dimZ() != (size_t)mDesc.C || host.dimB() != (size_t)mDesc.B)
        throw std::runtime_error("HipTensor::synchronizeHToD(): host tensor dimensions do not match");
    if (mDesc.halo != 0 && mDesc.layout != N2D2HIP_S2D)
        throw std::runtime_error("HipTensor::synchronizeHToD(): tensors with a halo are written by convolutions only");
    n2d2hip_tensor f = mDesc;
    f.dtype = N2D2HIP_F32;
    f.layout = N2D2HIP_NCHW;
    f.halo = 0;
    checkHip(hipMalloc(&f.data, host.size() * sizeof(float)), "HipTensor::synchronizeHToD(): hipMalloc");
    hipError_t e = hipMemcpy(f.data, host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice);
    int rc = N2D2HIP_OK;
    if (e == hipSuccess) {
        rc = n2d2hip_convert(&f, &mDesc, stream);
        e = hipStreamSynchronize((hipStream_t)stream);
    }
    (void)hipFree(f.data);
    checkHip(e, "HipTensor::synchronizeHToD()");
    checkStatus(rc);
    mHostValid = false;
}

// -------------------------------------------------------------------- Scaling
ScalingMode parseScalingMode(const std::string& str)
{
    // the spellings of include/ScalingMode.hpp
    if (str == "None") return ScalingMode::NONE;
    if (str == "Floating-point") return ScalingMode::FLOAT_MULT;
    if (str == "Fixed-point16") return ScalingMode::FIXED_MULT16;
    if (str == "Fixed-point32") return ScalingMode::FIXED_MULT32;
    if (str == "Single-shift") return ScalingMode::SINGLE_SHIFT;
    if (str == "Double-shift") return ScalingMode::DOUBLE_SHIFT;
    throw std::runtime_error("Unknown scaling mode \"" + str + "\"");
}

bool Scaling::allScalingsPositive() const
{
    switch (mMode) {
    case ScalingMode::FLOAT_MULT: return std::all_of(mFloat.begin(), mFloat.end(), [](Float_T v) { return v >= 0.0; });
    case ScalingMode::FIXED_MULT16:
    case ScalingMode::FIXED_MULT32: return std::all_of(mFixed.begin(), mFixed.end(), [](std::int32_t v) { return v >= 0; });
    case ScalingMode::SINGLE_SHIFT:
    case ScalingMode::DOUBLE_SHIFT: return true;
    default: throw std::runtime_error("Unsupported scaling mode");
    }
}

std::size_t Scaling::nbOutputs() const
{
    switch (mMode) {
    case ScalingMode::FLOAT_MULT: return mFloat.size();
    case ScalingMode::FIXED_MULT16:
    case ScalingMode::FIXED_MULT32: return mFixed.size();
    case ScalingMode::SINGLE_SHIFT: return mShift.size();
    case ScalingMode::DOUBLE_SHIFT: return mShift.size() / 2;
    default: return 0;
    }
}

// Builds the C-ABI object for "Scaling::propagate + activation" of one cell.
static n2d2hip_act_t makeAct(const Scaling& s, int kind, float leak, std::size_t nbBits, bool unsignedOut, unsigned int nbChannels,
                             const std::string& cellName)
{
    n2d2hip_activation d;
    std::memset(&d, 0, sizeof(d));
    d.kind = kind;
    d.leak_slope = leak;
    d.nb_bits = (int)nbBits;
    d.unsigned_out = unsignedOut ? 1 : 0;
    d.frac_bits = (int)s.getFractionalBits();
    d.is_clipped = s.getIsClipped() ? 1 : 0;
    d.clipping = s.getClippingPerOutput().empty() ? nullptr : s.getClippingPerOutput().data();
    switch (s.getMode()) {
    case ScalingMode::NONE: d.scaling_mode = N2D2HIP_SCALING_NONE; break;
    case ScalingMode::FLOAT_MULT: d.scaling_mode = N2D2HIP_SCALING_FLOAT_MULT; d.scaling = s.getFloatScalingPerOutput().data(); break;
    case ScalingMode::FIXED_MULT16: d.scaling_mode = N2D2HIP_SCALING_FIXED_MULT16; d.scaling = s.getFixedScalingPerOutput().data(); break;
    case ScalingMode::FIXED_MULT32: d.scaling_mode = N2D2HIP_SCALING_FIXED_MULT32; d.scaling = s.getFixedScalingPerOutput().data(); break;
    case ScalingMode::SINGLE_SHIFT: d.scaling_mode = N2D2HIP_SCALING_SINGLE_SHIFT; d.scaling = s.getShiftScalingPerOutput().data(); break;
    case ScalingMode::DOUBLE_SHIFT: d.scaling_mode = N2D2HIP_SCALING_DOUBLE_SHIFT; d.scaling = s.getShiftScalingPerOutput().data(); break;
    }
    if (s.getMode() != ScalingMode::NONE && s.nbOutputs() != nbChannels)
        throw std::runtime_error("Cell " + cellName + ": the scaling has " + std::to_string(s.nbOutputs()) + " entries for "
                                 + std::to_string(nbChannels) + " outputs");
    if (d.is_clipped && s.getClippingPerOutput().size() != nbChannels && s.getMode() != ScalingMode::SINGLE_SHIFT
        && s.getMode() != ScalingMode::DOUBLE_SHIFT)
        throw std::runtime_error("Cell " + cellName + ": clipping vector size does not match the number of outputs");
    n2d2hip_act_t h = nullptr;
    checkStatus(n2d2hip_act_create(&d, (int)nbChannels, &h));
    return h;
}

// ----------------------------------------------------------- static state
int CellExport::mPrecision = 0;
bool DeepNetExport::mUnsignedData = true;
bool DeepNetExport::mEnvDataUnsigned = false;

bool DeepNetExport::isCellOutputUnsigned(const Cell& cell)
{
    if (CellExport::mPrecision <= 0 || !DeepNetExport::mUnsignedData)
        return false;            // unsigned cells are not allowed
    return cell.getOutputsRange().first >= 0.0;
}

// ---------------------------------------------------------------- activations
const char* RectifierActivation::Type = "Rectifier";
const char* LinearActivation::Type = "Linear";

void RectifierActivation::setParameter(const std::string& name, double value)
{
    if (name == "LeakSlope") mLeakSlope = value;
    else if (name == "Clipping") mClipping = value;
    else throw std::runtime_error("Parameter does not exist: " + name);
    ++mRevision;
}
void LinearActivation::setParameter(const std::string& name, double value)
{
    if (name == "Clipping") mClipping = value;
    else throw std::runtime_error("Parameter does not exist: " + name);
    ++mRevision;
}

template <> Registrar<RectifierActivation> RectifierActivation_Frame_HIP<float>::mRegistrar(
    "Frame_HIP", RectifierActivation_Frame_HIP<float>::create, Registrar<RectifierActivation>::Type<float>());
template <> Registrar<LinearActivation> LinearActivation_Frame_HIP<float>::mRegistrar(
    "Frame_HIP", LinearActivation_Frame_HIP<float>::create, Registrar<LinearActivation>::Type<float>());

// ----------------------------------------------------------------------- Cell
std::pair<double, double> Cell::getOutputsRangeParents() const
{
    if (mParents.empty())
        throw std::runtime_error("Cell " + mName + " must have a parent.");
    std::pair<double, double> range;
    for (size_t i = 0; i < mParents.size(); ++i) {
        if (!mParents[i])
            throw std::runtime_error("Environment shouldn't be connected to cell " + mName + ".");
        const std::pair<double, double> r = mParents[i]->getOutputsRange();
        if (i == 0) range = r;
        else { range.first = std::min(range.first, r.first); range.second = std::max(range.second, r.second); }
    }
    return range;
}

Cell_Frame_HIP::~Cell_Frame_HIP()
{
    if (mActHandle)
        n2d2hip_act_destroy(mActHandle);
}

void Cell_Frame_HIP::addInput(Cell_Frame_HIP* parent)
{
    if (!parent)
        throw std::runtime_error("Cell " + mName + ": null parent");
    if (!mInputs.empty() && (parent->getOutputsWidth() != mInW || parent->getOutputsHeight() != mInH || parent->batchSize() != mBatch))
        throw std::runtime_error("Cell " + mName + ": inputs of different sizes");
    mParents.push_back(parent);
    mParentCells.push_back(parent);
    mInputs.push_back(&parent->mOutputs);
    if (mInputs.size() == 1)
        mNbChannels = parent->getNbOutputs();
    else if (parent->getNbOutputs() != mNbChannels)
        throw std::runtime_error("Cell " + mName + ": inputs with different numbers of channels are not supported by Frame_HIP");
    mInW = parent->getOutputsWidth();
    mInH = parent->getOutputsHeight();
    mBatch = parent->batchSize();
    setOutputsDims();
}

void Cell_Frame_HIP::addInput(HipTensor& stimuli, unsigned int nbChannels, unsigned int height, unsigned int width, unsigned int batchSize)
{
    if (!mInputs.empty())
        throw std::runtime_error("Cell " + mName + ": the environment must be the only input");
    mParents.push_back(nullptr);
    mParentCells.push_back(nullptr);
    mInputs.push_back(&stimuli);
    mNbChannels = nbChannels;
    mInW = width;
    mInH = height;
    mBatch = batchSize;
    setOutputsDims();
}

void Cell_Frame_HIP::addInputChannels(Cell_Frame_HIP* parent)
{
    if (!parent || mInputs.empty() || !mParentCells[0])
        throw std::runtime_error("Cell " + mName + ": several inputs must all be cells");
    if (parent->getOutputsWidth() != mInW || parent->getOutputsHeight() != mInH || parent->batchSize() != mBatch)
        throw std::runtime_error("Cell " + mName + ": inputs of different sizes");
    mParents.push_back(parent);
    mParentCells.push_back(parent);
    mInputs.push_back(&parent->mOutputs);
    mNbChannels += parent->getNbOutputs();
}

int Cell_Frame_HIP::prepareGathered()
{
    const int dtype = mInputs.at(0)->desc().dtype;
    for (const HipTensor* t : mInputs)
        if (t->desc().dtype != dtype)
            throw std::runtime_error("Cell " + mName + ": the inputs mix signed and unsigned outputs");
    if (mInputs.size() > 1) {
        // Several inputs are gathered into one tensor by an extra launch per forward (n2d2hip_concat_channels: every input
        // read once and written once more).  They must still be what the cell was given: one batch, one size.
        for (const HipTensor* t : mInputs)
            if (t->desc().B != (int)mBatch || t->desc().H != (int)mInH || t->desc().W != (int)mInW)
                throw std::runtime_error("Cell " + mName + ": an input is " + std::to_string(t->desc().B) + "x" + std::to_string(t->desc().H) + "x"
                                         + std::to_string(t->desc().W) + " (batch x height x width), the cell was given " + std::to_string(mBatch)
                                         + "x" + std::to_string(mInH) + "x" + std::to_string(mInW));
        const n2d2hip_tensor& g = mGathered.desc();
        if (mGathered.empty() || g.dtype != dtype || g.C != (int)mNbChannels || g.B != (int)mBatch || g.H != (int)mInH || g.W != (int)mInW)
            mGathered.resize((int)mBatch, (int)mNbChannels, (int)mInH, (int)mInW, dtype);
    }
    return dtype;
}

const n2d2hip_tensor& Cell_Frame_HIP::gatherInputs()
{
    std::vector<const n2d2hip_tensor*> ins;
    for (const HipTensor* t : mInputs)
        ins.push_back(&t->desc());
    checkStatus(n2d2hip_concat_channels((int)ins.size(), ins.data(), &mGathered.desc(), mStream));
    return mGathered.desc();
}

void Cell_Frame_HIP::clearInputs()
{
    mInputs.clear();
    mParentCells.clear();
    mParents.clear();
    mNbChannels = 0;
    mInW = mInH = 0;
}

void Cell_Frame_HIP::replaceInput(HipTensor& oldInputs, HipTensor& newInputs, Cell_Frame_HIP* newParent)
{
    unsigned int C, H, W, B;
    if (newParent) {
        if (&newParent->mOutputs != &newInputs)
            throw std::runtime_error("Cell_Frame::replaceInput(): the new input is not the output of the cell given as its producer.");
        C = newParent->getNbOutputs();
        H = newParent->getOutputsHeight();
        W = newParent->getOutputsWidth();
        B = newParent->batchSize();
    } else {
        if (newInputs.empty())
            throw std::runtime_error("Cell_Frame::replaceInput(): the new input is empty.");
        const n2d2hip_tensor& d = newInputs.desc();
        C = (unsigned int)d.C;
        H = (unsigned int)d.H;
        W = (unsigned int)d.W;
        B = (unsigned int)d.B;
    }
    size_t pos = mInputs.size();
    for (size_t i = 0; i < mInputs.size() && pos == mInputs.size(); ++i)
        if (mInputs[i] == &oldInputs)
            pos = i;
    if (pos == mInputs.size())
        throw std::runtime_error("Cell_Frame::replaceInput(): can't replace input, the input has not been found.");
    if (mInputs.size() > 1 && (C != mNbChannels || B != mBatch))
        throw std::runtime_error("Cell_Frame::replaceInput(): can't replace input, the new input does not match the other inputs!");
    const unsigned int oldC = mNbChannels, oldB = mBatch, oldInW = mInW, oldInH = mInH, oldW = mOutW, oldH = mOutH;
    mNbChannels = C;
    mBatch = B;
    mInW = W;
    mInH = H;
    setOutputsDims();
    if (mInputs.size() > 1 && (mOutW != oldW || mOutH != oldH)) {
        mNbChannels = oldC;
        mBatch = oldB;
        mInW = oldInW;
        mInH = oldInH;
        setOutputsDims();
        throw std::runtime_error("Cell_Frame::replaceInput(): can't replace input, the output dimension has changed and doesn't"
                                 " match the other inputs!");
    }
    mInputs[pos] = &newInputs;
    mParentCells[pos] = newParent;
    mParents[pos] = newParent;
}

void Cell_Frame_HIP::backPropagate()
{
    throw std::runtime_error("Cell " + mName + ": the cells of the model \"Frame_HIP\" run quantized inference and have no backPropagate();"
                             " learn with the model \"Frame_HIP_QAT\"");
}

void Cell_Frame_HIP::update()
{
    throw std::runtime_error("Cell " + mName + ": the cells of the model \"Frame_HIP\" run quantized inference and have no update();"
                             " learn with the model \"Frame_HIP_QAT\"");
}

void Cell_Frame_HIP::checkGradient(double /*epsilon*/, double /*maxError*/)
{
    throw std::runtime_error("Cell " + mName + ": the cells of the model \"Frame_HIP\" run quantized inference and have no gradient to check");
}

unsigned int Cell_Frame_HIP::getMaxOutput(unsigned int batchPos)
{
    const Tensor<Float_T>& out = getOutputs();
    if (batchPos >= out.dimB())
        throw std::runtime_error("Cell " + mName + ": getMaxOutput(): batch position out of range");
    const size_t n = out.dimX() * out.dimY() * out.dimZ();
    const Float_T* p = out.data() + (size_t)batchPos * n;
    return (unsigned int)std::distance(p, std::max_element(p, p + n));
}

const Tensor<Float_T>& Cell_Frame_HIP::getOutputs()
{
    if (mFoldedInto)
        throw std::runtime_error("Cell " + mName + ": its output is not materialised, cell " + mFoldedInto->getName()
                                 + " computes it on the fly (DeepNet::setFusion(false) keeps every output)");
    return mOutputs.synchronizeDToH(mStream);
}

int Cell_Frame_HIP::outputDType(const Scaling* standalone) const
{
    const Scaling* s = standalone ? standalone : (mActivation ? &mActivation->getActivationScaling() : nullptr);
    if (!s || s->getMode() == ScalingMode::NONE)
        return N2D2HIP_I32;
    return DeepNetExport::isCellOutputUnsigned(*this) ? N2D2HIP_U8B : N2D2HIP_I8;
}

void Cell_Frame_HIP::allocateOutputs(const Scaling* standalone)
{
    if (mInputs.empty())
        throw std::runtime_error("Cell " + mName + " has no input");
    mOutputs.resize((int)mBatch, (int)mNbOutputs, (int)mOutH, (int)mOutW, outputDType(standalone), mOutputsHalo);
}

void Cell_Frame_HIP::setOutputsHalo(int halo)
{
    if (halo == mOutputsHalo)
        return;
    mOutputsHalo = halo;
    if (!mOutputs.empty())
        mOutputs.resize(mOutputs.desc().B, mOutputs.desc().C, mOutputs.desc().H, mOutputs.desc().W, mOutputs.desc().dtype, halo);
}

n2d2hip_act_t Cell_Frame_HIP::activationHandle(const Scaling* standalone)
{
    const bool uns = DeepNetExport::isCellOutputUnsigned(*this);
    const unsigned rev = mActivation ? mActivation->revision() : 0u;
    if (mActHandle && mActRevision == rev && mActUnsigned == (int)uns && !standalone)
        return mActHandle;
    if (mActHandle) {
        n2d2hip_act_destroy(mActHandle);
        mActHandle = nullptr;
    }
    Scaling none;
    const Scaling& s = standalone ? *standalone : (mActivation ? mActivation->getActivationScaling() : none);
    // RectifierActivation_Frame.hpp:65-66: the activation's bit width when set, else the cell's
    const std::size_t nbBits = (mActivation && mActivation->getQuantizedNbBits() > 0) ? mActivation->getQuantizedNbBits() : mQuantizedNbBits;
    const int kind = (mActivation && !standalone) ? mActivation->abiKind() : N2D2HIP_ACT_LINEAR;
    const float leak = (mActivation && !standalone) ? mActivation->leakSlope() : 0.0f;
    mActHandle = makeAct(s, kind, leak, nbBits, uns, mNbOutputs, mName);
    ++mActGeneration;
    mActRevision = rev;
    mActUnsigned = (int)uns;
    // the storage type follows the signedness decision
    if (mOutputs.empty() || mOutputs.desc().dtype != outputDType(standalone))
        allocateOutputs(standalone);
    return mActHandle;
}

// Integer check of a float parameter on its way to the device.
static long long toInteger(Float_T v, long long lo, long long hi, const std::string& what)
{
    const double r = std::nearbyint((double)v);
    if (r != (double)v || r < (double)lo || r > (double)hi) {
        std::ostringstream msg;
        msg << what << ": value " << v << " is not an integer in [" << lo << "," << hi << "]; quantize the network before running it on Frame_HIP";
        throw std::runtime_error(msg.str());
    }
    return (long long)r;
}

static std::vector<unsigned char> packWeights(const Tensor<Float_T>& w, int bits, const std::string& name)
{
    const long long lo = bits == 4 ? -8 : -128, hi = bits == 4 ? 7 : 127;
    std::vector<unsigned char> out(bits == 4 ? (w.size() + 1) / 2 : w.size(), 0);
    for (size_t i = 0; i < w.size(); ++i) {
        const long long v = toInteger(w(i), lo, hi, "Cell " + name + " weights");
        if (bits == 4)
            out[i >> 1] |= (unsigned char)((v & 15) << ((i & 1) ? 4 : 0));
        else
            out[i] = (unsigned char)(signed char)v;
    }
    return out;
}

// ------------------------------------------------------------------- ConvCell
const char* ConvCell::Type = "Conv";

ConvCell::ConvCell(const std::vector<unsigned int>& kernelDims, const std::vector<unsigned int>& subSampleDims,
                   const std::vector<unsigned int>& strideDims, const std::vector<int>& paddingDims,
                   const std::vector<unsigned int>& dilationDims)
    : mKernelDims(kernelDims), mSubSampleDims(subSampleDims), mStrideDims(strideDims), mDilationDims(dilationDims),
      mPaddingDims(paddingDims), mNoBias(false), mNbGroups(1), mWeightBits(8), mDirty(true)
{
    if (mKernelDims.size() != 2)
        throw std::runtime_error("ConvCell: only 2D convolutions are supported by Frame_HIP");
    if (mSubSampleDims.empty()) mSubSampleDims.assign(2, 1U);
    if (mStrideDims.empty()) mStrideDims.assign(2, 1U);
    if (mPaddingDims.empty()) mPaddingDims.assign(2, 0);
    if (mDilationDims.empty()) mDilationDims.assign(2, 1U);
    if (mSubSampleDims.size() != 2 || mSubSampleDims[0] < 1 || mSubSampleDims[1] < 1)
        throw std::runtime_error("ConvCell: SubSampleDims must be two positive values");
}

void ConvCell::setParameter(const std::string& name, bool value)
{
    if (name == "NoBias") { mNoBias = value; mDirty = true; }
    else throw std::runtime_error("Parameter does not exist: " + name);
}

template <class T>
ConvCell_Frame_HIP<T>::ConvCell_Frame_HIP(const DeepNet& /*deepNet*/, const std::string& name, const std::vector<unsigned int>& kernelDims,
                                          unsigned int nbOutputs, const std::vector<unsigned int>& subSampleDims,
                                          const std::vector<unsigned int>& strideDims, const std::vector<int>& paddingDims,
                                          const std::vector<unsigned int>& dilationDims, const std::shared_ptr<Activation>& activation)
    : Cell(name, nbOutputs), ConvCell(kernelDims, subSampleDims, strideDims, paddingDims, dilationDims), mConv(nullptr), mConvActGen(0), mConvInDType(-1),
      mDwPw(nullptr), mFusedDw(nullptr)
{
    mActivation = activation;
}

template <class T>
ConvCell_Frame_HIP<T>::~ConvCell_Frame_HIP()
{
    if (mDwPw) n2d2hip_dw_pw_destroy(mDwPw);
    if (mConv) n2d2hip_conv_destroy(mConv);
}

template <class T>
bool ConvCell_Frame_HIP<T>::fuseDepthwise(Cell_Frame_HIP* depthwise)
{
    if (mDwPw || !mConv || !depthwise || !depthwise->convHandle() || depthwise->foldedInto() || foldedInto() || mInputs.size() != 1
        || depthwise->parentCells().size() != 1 || depthwise->inputTensor(0)->desc().halo != 0)
        return false;
    n2d2hip_dw_pw_t fused = nullptr;
    const int rc = n2d2hip_dw_pw_create(depthwise->convHandle(), mConv, &fused);
    if (rc == N2D2HIP_ERR_UNSUPPORTED)
        return false;
    checkStatus(rc);
    const n2d2hip_tensor& x = depthwise->inputTensor(0)->desc();
    if (!n2d2hip_dw_pw_pays(fused, x.B, x.H, x.W)) {
        n2d2hip_dw_pw_destroy(fused);
        return false;
    }
    mDwPw = fused;
    mFusedDw = depthwise;
    depthwise->setFoldedInto(this);
    return true;
}

template <class T>
void ConvCell_Frame_HIP<T>::clearFusion()
{
    if (mDwPw) {
        n2d2hip_dw_pw_destroy(mDwPw);
        mDwPw = nullptr;
        mFusedDw->setFoldedInto(nullptr);
        mFusedDw = nullptr;
    }
}

template <class T>
void ConvCell_Frame_HIP<T>::setOutputsDims()
{
    // src/Cell/ConvCell.cpp:1169-1195
    const unsigned int in[2] = {mInW, mInH};
    unsigned int out[2];
    for (int dim = 0; dim < 2; ++dim) {
        const int kernelExtent = (int)(mDilationDims[dim] * (mKernelDims[dim] - 1) + 1);
        out[dim] = (unsigned int)std::ceil(std::floor(((int)in[dim] + 2 * mPaddingDims[dim] - kernelExtent + (int)mStrideDims[dim])
                                                      / (double)mStrideDims[dim]) / (double)mSubSampleDims[dim]);
    }
    mOutW = out[0];
    mOutH = out[1];
}

template <class T>
void ConvCell_Frame_HIP<T>::addInput(Cell_Frame_HIP* parent)
{
    if (mInputs.empty())
        Cell_Frame_HIP::addInput(parent);
    else
        addInputChannels(parent);
    mDirty = true;
}

template <class T>
void ConvCell_Frame_HIP<T>::initialize()
{
    if (mInputs.empty())
        throw std::runtime_error("ConvCell_Frame_HIP " + mName + ": no input");
    allocateOutputs();
}

template <class T>
void ConvCell_Frame_HIP<T>::propagate(bool /*inference*/)
{
    prepare();
    launch();
}

template <class T>
void ConvCell_Frame_HIP<T>::launch()
{
    if (mDwPw)
        checkStatus(n2d2hip_dw_pw_forward(mDwPw, &mFusedDw->inputTensor(0)->desc(), &mOutputs.desc(), mStream));
    else if (mInputs.size() > 1)
        checkStatus(n2d2hip_conv_forward(mConv, &gatherInputs(), &mOutputs.desc(), mStream));
    else
        checkStatus(n2d2hip_conv_forward(mConv, &mInputs[0]->desc(), &mOutputs.desc(), mStream));
    mOutputs.invalidateHost();
}

template <class T>
bool ConvCell_Frame_HIP<T>::prepare()
{
    n2d2hip_act_t act = activationHandle();
    const int inDType = prepareGathered();
    bool rebuilt = false;
    if (mDirty || activationGeneration() != mConvActGen || !mConv || inDType != mConvInDType) {
        clearFusion();
        if (mConv) { n2d2hip_conv_destroy(mConv); mConv = nullptr; }
        const unsigned int cg = weightSlices();
        if (mWeights.dimX() != mKernelDims[0] || mWeights.dimY() != mKernelDims[1] || mWeights.dimZ() != cg || mWeights.dimB() != mNbOutputs)
            throw std::runtime_error("ConvCell_Frame_HIP " + mName + ": weights must be {kW, kH, nbChannels/groups, nbOutputs}");
        if (hasIrregularMapping() && mInputs.size() > 1)
            throw std::runtime_error("ConvCell_Frame_HIP " + mName + ": an irregular connection map over several inputs is not supported");
        n2d2hip_conv_desc d = {};
        d.C = (int)mNbChannels; d.O = (int)mNbOutputs; d.kW = (int)mKernelDims[0]; d.kH = (int)mKernelDims[1];
        d.strideX = (int)mStrideDims[0]; d.strideY = (int)mStrideDims[1];
        d.padL = d.padR = mPaddingDims[0]; d.padT = d.padB = mPaddingDims[1];
        d.dilX = (int)mDilationDims[0]; d.dilY = (int)mDilationDims[1];
        // an irregular map runs as a full connection whose missing connections weigh nothing
        d.groups = hasIrregularMapping() ? 1 : (int)mNbGroups; d.weight_bits = mWeightBits;
        d.subX = (int)mSubSampleDims[0]; d.subY = (int)mSubSampleDims[1];
        const std::vector<unsigned char> w = packWeights(hasIrregularMapping() ? fullConnectionWeights() : mWeights, mWeightBits, mName);
        std::vector<std::int32_t> b;
        if (!mNoBias) {
            if (mBias.size() != mNbOutputs)
                throw std::runtime_error("ConvCell_Frame_HIP " + mName + ": one bias per output expected");
            for (size_t i = 0; i < mBias.size(); ++i)
                b.push_back((std::int32_t)toInteger(mBias(i), std::numeric_limits<std::int32_t>::min(), std::numeric_limits<std::int32_t>::max(),
                                                    "Cell " + mName + " biases"));
        }
        checkStatus(n2d2hip_conv_create(&d, w.data(), mNoBias ? nullptr : b.data(), act, inDType, &mConv));
        mConvActGen = activationGeneration();
        mConvInDType = inDType;
        mDirty = false;
        rebuilt = true;
    }
    return rebuilt;
}

template <> Registrar<ConvCell> ConvCell_Frame_HIP<float>::mRegistrar("Frame_HIP", ConvCell_Frame_HIP<float>::create,
                                                                      Registrar<ConvCell>::Type<float>());

// --------------------------------------------------------------------- FcCell
const char* FcCell::Type = "Fc";

void FcCell::setParameter(const std::string& name, bool value)
{
    if (name == "NoBias") { mNoBias = value; mDirty = true; }
    else throw std::runtime_error("Parameter does not exist: " + name);
}

template <class T>
FcCell_Frame_HIP<T>::FcCell_Frame_HIP(const DeepNet& /*deepNet*/, const std::string& name, unsigned int nbOutputs,
                                      const std::shared_ptr<Activation>& activation)
    : Cell(name, nbOutputs), mFc(nullptr), mFcActGen(0), mFcNbInputs(0)
{
    mActivation = activation;
}

template <class T>
FcCell_Frame_HIP<T>::~FcCell_Frame_HIP()
{
    if (mChain) n2d2hip_fc_chain_destroy(mChain);
    if (mFc) n2d2hip_fc_destroy(mFc);
}

template <class T>
bool FcCell_Frame_HIP<T>::fuseChain(const std::vector<FcCell_Frame_HIP<T>*>& earlier)
{
    if (mChain || earlier.empty() || !mFc || mInputs.size() != 1)
        return false;
    std::vector<n2d2hip_fc_t> cells;
    for (FcCell_Frame_HIP<T>* c : earlier) {
        if (!c || !c->mFc || c->foldedInto() || c->mChain || c->mInputs.size() != 1)
            return false;
        cells.push_back(c->mFc);
    }
    cells.push_back(mFc);
    if (n2d2hip_fc_chain_create((int)cells.size(), cells.data(), &mChain) != N2D2HIP_OK) {
        mChain = nullptr;
        return false;
    }
    mChained = earlier;
    for (FcCell_Frame_HIP<T>* c : mChained)
        c->setFoldedInto(this);
    return true;
}

template <class T>
void FcCell_Frame_HIP<T>::clearFusion()
{
    if (mChain) {
        n2d2hip_fc_chain_destroy(mChain);
        mChain = nullptr;
        for (FcCell_Frame_HIP<T>* c : mChained)
            c->setFoldedInto(nullptr);
        mChained.clear();
    }
}

template <class T>
void FcCell_Frame_HIP<T>::setOutputsDims()
{
    mOutW = 1;
    mOutH = 1;
}

template <class T>
void FcCell_Frame_HIP<T>::addInput(Cell_Frame_HIP* parent)
{
    if (mInputs.empty())
        Cell_Frame_HIP::addInput(parent);
    else
        addInputChannels(parent);
    mDirty = true;
}

template <class T>
void FcCell_Frame_HIP<T>::initialize()
{
    if (mInputs.empty())
        throw std::runtime_error("FcCell_Frame_HIP " + mName + ": no input");
    allocateOutputs();
}

template <class T>
void FcCell_Frame_HIP<T>::propagate(bool /*inference*/)
{
    prepare();
    launch();
}

template <class T>
void FcCell_Frame_HIP<T>::launch()
{
    if (mChain)
        checkStatus(n2d2hip_fc_chain_forward(mChain, &mChained[0]->mInputs[0]->desc(), &mOutputs.desc(), mStream));
    else
        checkStatus(n2d2hip_fc_forward(mFc, mInputs.size() > 1 ? &gatherInputs() : &mInputs[0]->desc(), &mOutputs.desc(), mStream));
    mOutputs.invalidateHost();
}

template <class T>
bool FcCell_Frame_HIP<T>::prepare()
{
    n2d2hip_act_t act = activationHandle();
    const int inDType = prepareGathered();
    bool rebuilt = false;
    if (mDirty || activationGeneration() != mFcActGen || !mFc || mFcNbInputs != mInputs.size() || inDType != mFcInDType) {
        clearFusion();
        if (mFc) { n2d2hip_fc_destroy(mFc); mFc = nullptr; }
        const size_t K = (size_t)mNbChannels * mInH * mInW;
        if (mWeights.size() != K * mNbOutputs)
            throw std::runtime_error("FcCell_Frame_HIP " + mName + ": weights must hold nbOutputs x (channels*height*width) values");
        const std::vector<unsigned char> w = packWeights(mWeights, 8, mName);
        std::vector<std::int32_t> b;
        if (!mNoBias) {
            if (mBias.size() != mNbOutputs)
                throw std::runtime_error("FcCell_Frame_HIP " + mName + ": one bias per output expected");
            // every input's inner product starts from the bias (src/Cell/FcCell_Frame.cpp:309) and the products are added up
            const long long n = (long long)mInputs.size();
            for (size_t i = 0; i < mBias.size(); ++i) {
                const long long one = toInteger(mBias(i), std::numeric_limits<std::int32_t>::min(), std::numeric_limits<std::int32_t>::max(),
                                                "Cell " + mName + " biases");
                if (one * n < std::numeric_limits<std::int32_t>::min() || one * n > std::numeric_limits<std::int32_t>::max())
                    throw std::runtime_error("FcCell_Frame_HIP " + mName + ": the bias, added once per input, leaves 32 bits");
                b.push_back((std::int32_t)(one * n));
            }
        }
        checkStatus(n2d2hip_fc_create((int)mNbChannels, (int)mInH, (int)mInW, (int)mNbOutputs, 8, w.data(), mNoBias ? nullptr : b.data(), act,
                                      inDType, &mFc));
        mFcActGen = activationGeneration();
        mFcNbInputs = mInputs.size();
        mFcInDType = inDType;
        mDirty = false;
        rebuilt = true;
    }
    return rebuilt;
}

template <> Registrar<FcCell> FcCell_Frame_HIP<float>::mRegistrar("Frame_HIP", FcCell_Frame_HIP<float>::create, Registrar<FcCell>::Type<float>());

// ------------------------------------------------------------------- PoolCell
const char* PoolCell::Type = "Pool";

template <class T>
PoolCell_Frame_HIP<T>::PoolCell_Frame_HIP(const DeepNet& /*deepNet*/, const std::string& name, const std::vector<unsigned int>& poolDims,
                                          unsigned int nbOutputs, const std::vector<unsigned int>& strideDims,
                                          const std::vector<unsigned int>& paddingDims, Pooling pooling,
                                          const std::shared_ptr<Activation>& activation)
    : Cell(name, nbOutputs), PoolCell(poolDims, strideDims, paddingDims, pooling)
{
    if (mPoolDims.size() != 2)
        throw std::runtime_error("PoolCell: only 2D pooling is supported by Frame_HIP");
    if (mStrideDims.empty()) mStrideDims.assign(2, 1U);
    if (mPaddingDims.empty()) mPaddingDims.assign(2, 0U);
    mActivation = activation;
    if (activation)
        throw std::runtime_error("PoolCell_Frame_HIP " + name + ": an activation on a pooling cell is not supported");
}

template <class T>
void PoolCell_Frame_HIP<T>::setOutputsDims()
{
    // src/Cell/PoolCell.cpp:219-240
    mOutW = (unsigned int)((mInW + 2 * mPaddingDims[0] - mPoolDims[0] + mStrideDims[0]) / (double)mStrideDims[0]);
    mOutH = (unsigned int)((mInH + 2 * mPaddingDims[1] - mPoolDims[1] + mStrideDims[1]) / (double)mStrideDims[1]);
}

template <class T>
void PoolCell_Frame_HIP<T>::addInput(Cell_Frame_HIP* parent)
{
    if (mInputs.empty())
        Cell_Frame_HIP::addInput(parent);
    else
        addInputChannels(parent);
}

template <class T>
void PoolCell_Frame_HIP<T>::setMapping(const Tensor<bool>& map)
{
    if (map.dimX() != mNbOutputs || map.dimY() != mNbChannels)
        throw std::runtime_error("PoolCell_Frame_HIP::setMapping(): the map of " + mName + " must be {nbOutputs, nbChannels}");
    bool unit = mNbOutputs == mNbChannels;
    for (std::size_t o = 0; unit && o < mNbOutputs; ++o)
        for (std::size_t ch = 0; unit && ch < mNbChannels; ++ch)
            unit = map.at(o, ch) == (o == ch);
    mMapping = unit ? Tensor<bool>() : map;
    if (mMappingDevice) {
        (void)hipFree(mMappingDevice);
        mMappingDevice = nullptr;
    }
    // a pooling over a map is a launch of its own: the first convolution, if it was computing this pooling, runs again
    if (!unit)
        clearFusion();
}

template <class T>
PoolCell_Frame_HIP<T>::~PoolCell_Frame_HIP()
{
    if (mMappingDevice) (void)hipFree(mMappingDevice);
}

template <class T>
void PoolCell_Frame_HIP<T>::initialize()
{
    if (mInputs.empty())
        throw std::runtime_error("PoolCell_Frame_HIP " + mName + ": no input");
    if (mMapping.empty() && mNbOutputs != mNbChannels)
        throw std::runtime_error("PoolCell_Frame_HIP " + mName + ": without a connection map (setMapping) the cell pools one output per "
                                 "channel, NbOutputs must be the inputs' channels");
    uploadMapping();
    mOutputs.resize((int)mBatch, (int)mNbOutputs, (int)mOutH, (int)mOutW, mInputs[0]->desc().dtype);
}

// Checks the connection map against the cell as it stands now (inputs may have been added since setMapping) and copies it
// to the device.  Called by initialize(), and by propagate() when a map was set behind initialize().
template <class T>
void PoolCell_Frame_HIP<T>::uploadMapping()
{
    if (mMappingDevice) {
        (void)hipFree(mMappingDevice);
        mMappingDevice = nullptr;
    }
    if (mMapping.empty())
        return;
    if (mMapping.dimX() != mNbOutputs || mMapping.dimY() != mNbChannels)
        throw std::runtime_error("PoolCell_Frame_HIP " + mName + ": the connection map is {" + std::to_string(mMapping.dimX()) + ", "
                                 + std::to_string(mMapping.dimY()) + "}, the cell has " + std::to_string(mNbOutputs) + " outputs and "
                                 + std::to_string(mNbChannels) + " channels (inputs added after setMapping?)");
    // channels of one input only behind every output
    for (std::size_t o = 0; o < mNbOutputs; ++o) {
        int owner = -1;
        std::size_t first = 0;
        for (std::size_t k = 0; k < mInputs.size(); ++k) {
            const std::size_t n = (std::size_t)mInputs[k]->desc().C;
            for (std::size_t ch = first; ch < first + n; ++ch)
                if (mMapping.at(o, ch)) {
                    if (owner >= 0 && owner != (int)k)
                        throw std::runtime_error("PoolCell_Frame_HIP " + mName + ": an output that pools channels of several inputs is not supported");
                    owner = (int)k;
                }
            first += n;
        }
    }
    std::vector<unsigned char> host(mNbOutputs * mNbChannels);
    for (std::size_t o = 0; o < mNbOutputs; ++o)
        for (std::size_t ch = 0; ch < mNbChannels; ++ch)
            host[o * mNbChannels + ch] = mMapping.at(o, ch) ? 1 : 0;
    checkHip(hipMalloc((void**)&mMappingDevice, host.size()), "PoolCell_Frame_HIP::uploadMapping(): hipMalloc");
    checkHip(hipMemcpy(mMappingDevice, host.data(), host.size(), hipMemcpyHostToDevice), "PoolCell_Frame_HIP::uploadMapping(): hipMemcpy");
}

template <class T>
n2d2hip_pool_desc PoolCell_Frame_HIP<T>::poolDesc() const
{
    n2d2hip_pool_desc d;
    d.pooling = mPooling == Max ? N2D2HIP_POOL_MAX : N2D2HIP_POOL_AVERAGE;
    d.poolW = (int)mPoolDims[0]; d.poolH = (int)mPoolDims[1];
    d.strideX = (int)mStrideDims[0]; d.strideY = (int)mStrideDims[1];
    d.padX = (int)mPaddingDims[0]; d.padY = (int)mPaddingDims[1];
    return d;
}

template <class T>
bool PoolCell_Frame_HIP<T>::fuseFirstConv(Cell_Frame_HIP* conv)
{
    if (mFusedConv || !mMapping.empty() || !conv || !conv->convHandle() || conv->foldedInto() || mInputs.size() != 1 || conv->parentCells().size() != 1)
        return false;
    const n2d2hip_pool_desc d = poolDesc();
    const n2d2hip_tensor& x = conv->inputTensor(0)->desc();
    // (a space-to-depth input is the network's: its border is part of its form, and the library takes the pair on both forms
    // or says so when the launch is planned)
    if ((x.halo != 0 && x.layout != N2D2HIP_S2D) || !n2d2hip_conv_accepts_maxpool(conv->convHandle(), &d, x.H, x.W))
        return false;
    mFusedConv = conv;
    conv->setFoldedInto(this);
    return true;
}

template <class T>
bool PoolCell_Frame_HIP<T>::writesHalo() const
{
    if (mFusedConv)
        return true;
    if (mInputs.size() != 1 || mInputs[0]->empty() || !mMapping.empty())
        return false;
    const n2d2hip_pool_desc d = poolDesc();
    const n2d2hip_tensor& x = mInputs[0]->desc();
    return x.halo == 0 && n2d2hip_pool_writes_halo(&d, x.H, x.W, x.cs) != 0;
}

template <class T>
void PoolCell_Frame_HIP<T>::clearFusion()
{
    if (mFusedConv) {
        mFusedConv->setFoldedInto(nullptr);
        mFusedConv = nullptr;
    }
}

template <class T>
void PoolCell_Frame_HIP<T>::propagate(bool /*inference*/)
{
    const int dtype = prepareGathered();
    if (mOutputs.empty() || mOutputs.desc().dtype != dtype || mOutputs.desc().halo != mOutputsHalo)
        mOutputs.resize((int)mBatch, (int)mNbOutputs, (int)mOutH, (int)mOutW, dtype, mOutputsHalo);
    const n2d2hip_pool_desc d = poolDesc();
    // a map set behind initialize() (setMapping drops the device copy) is checked and copied now
    if (!mMapping.empty() && !mMappingDevice)
        uploadMapping();
    if (mFusedConv && mMapping.empty())
        checkStatus(n2d2hip_conv_forward_maxpool(mFusedConv->convHandle(), &d, &mFusedConv->inputTensor(0)->desc(), &mOutputs.desc(), mStream));
    else if (!mMapping.empty())
        checkStatus(n2d2hip_pool_forward_mapped(&d, mMappingDevice, (int)mNbOutputs, (int)mNbChannels,
                                                mInputs.size() > 1 ? &gatherInputs() : &mInputs[0]->desc(), &mOutputs.desc(), mStream));
    else
        checkStatus(n2d2hip_pool_forward(&d, mInputs.size() > 1 ? &gatherInputs() : &mInputs[0]->desc(), &mOutputs.desc(), mStream));
    mOutputs.invalidateHost();
}

template <> Registrar<PoolCell> PoolCell_Frame_HIP<float>::mRegistrar("Frame_HIP", PoolCell_Frame_HIP<float>::create,
                                                                      Registrar<PoolCell>::Type<float>());

// --------------------------------------------------------------- ElemWiseCell
const char* ElemWiseCell::Type = "ElemWise";

std::pair<double, double> ElemWiseCell::elemWiseOutputsRange() const
{
    const std::pair<double, double> parents = getOutputsRangeParents();
    const double inf = std::numeric_limits<double>::infinity();
    if (mOperation == EuclideanSum)
        return std::make_pair(0.0, inf);
    if (parents.first >= 0.0) {
        const bool shiftsPos = std::all_of(mShifts.begin(), mShifts.end(), [](Float_T v) { return v >= 0.0; });
        const bool weightsPos = std::all_of(mWeights.begin(), mWeights.end(), [](Float_T v) { return v >= 0.0; });
        if (mOperation == Sum && shiftsPos && weightsPos) return std::make_pair(0.0, inf);
        if (mOperation == AbsSum && weightsPos) return std::make_pair(0.0, inf);
        if (mOperation == Prod || mOperation == Max) return std::make_pair(0.0, inf);
    }
    return std::make_pair(-inf, inf);
}

ElemWiseCell_Frame_HIP::ElemWiseCell_Frame_HIP(const DeepNet& /*deepNet*/, const std::string& name, unsigned int nbOutputs, Operation operation,
                                               CoeffMode mode, const std::vector<Float_T>& weights, const std::vector<Float_T>& shifts,
                                               const std::shared_ptr<Activation>& activation)
    : Cell(name, nbOutputs), ElemWiseCell(operation, mode, weights, shifts), mEw(nullptr), mEwActGen(0), mFusedConv(nullptr), mFusedIndex(0)
{
    mActivation = activation;
    if (operation != Sum)
        throw std::runtime_error("ElemWiseCell_Frame_HIP " + name + ": only the Sum operation is on the quantized path");
}

ElemWiseCell_Frame_HIP::~ElemWiseCell_Frame_HIP()
{
    if (mEw) n2d2hip_elemwise_destroy(mEw);
}

void ElemWiseCell_Frame_HIP::setOutputsDims()
{
    mOutW = mInW;
    mOutH = mInH;
}

void ElemWiseCell_Frame_HIP::initialize()
{
    if (mNbOutputs != mNbChannels)
        throw std::runtime_error("ElemWiseCell_Frame_HIP " + mName + ": the number of output channels must be equal to the sum of inputs channels.");
    // src/Cell/ElemWiseCell_Frame.cpp:75-87: default 1.0 / 0.0, one entry per input (per channel when PerChannel)
    const size_t n = mCoeffMode == PerChannel ? (size_t)mNbChannels : mInputs.size();
    mWeights.resize(n, 1.0f);
    mShifts.resize(n, 0.0f);
    allocateOutputs();
}

void ElemWiseCell_Frame_HIP::propagate(bool /*inference*/)
{
    prepare();
    launch();
}

bool ElemWiseCell_Frame_HIP::prepare()
{
    n2d2hip_act_t act = activationHandle();
    if (mEw && activationGeneration() == mEwActGen)
        return false;
    // the convolution that took this sum over borrows mEw: release it first
    clearFusion();
    if (mEw) { n2d2hip_elemwise_destroy(mEw); mEw = nullptr; }
    const int mode = mCoeffMode == PerChannel ? N2D2HIP_COEFF_PER_CHANNEL : (mCoeffMode == PerInput ? N2D2HIP_COEFF_PER_INPUT : N2D2HIP_COEFF_PER_LAYER);
    checkStatus(n2d2hip_elemwise_create((int)mInputs.size(), (int)mNbOutputs, mode, mWeights.data(), mShifts.data(), act, &mEw));
    mEwActGen = activationGeneration();
    return true;
}

// The tensor input k is read from: the ScalingCell's own input once that cell is folded
static HipTensor* sourceOf(const std::vector<Cell_Frame_HIP*>& folded, const std::vector<HipTensor*>& inputs, size_t k)
{
    return (k < folded.size() && folded[k]) ? folded[k]->inputTensor(0) : inputs[k];
}

void ElemWiseCell_Frame_HIP::launch()
{
    if (mBottleneck) {
        checkStatus(n2d2hip_bottleneck_forward(mBottleneck, &mBottleneckIn->getDeviceOutputs().desc(), &mOutputs.desc(), mStream));
    } else if (mChainConv) {
        checkStatus(n2d2hip_conv_chain_forward(mChainConv->convHandle(), mFusedConv->convHandle(), &mChainConv->inputTensor(0)->desc(),
                                               &sourceOf(mFoldedScaling, mInputs, 1 - mFusedIndex)->desc(), &mOutputs.desc(), mStream));
    } else if (mFusedConv) {
        checkStatus(n2d2hip_conv_forward_sum(mFusedConv->convHandle(), &mFusedConv->inputTensor(0)->desc(),
                                             &sourceOf(mFoldedScaling, mInputs, 1 - mFusedIndex)->desc(), &mOutputs.desc(), mStream));
    } else {
        std::vector<const n2d2hip_tensor*> ins;
        for (size_t k = 0; k < mInputs.size(); ++k)
            ins.push_back(&sourceOf(mFoldedScaling, mInputs, k)->desc());
        checkStatus(n2d2hip_elemwise_forward(mEw, ins.data(), &mOutputs.desc(), mStream));
    }
    mOutputs.invalidateHost();
}

bool ElemWiseCell_Frame_HIP::foldInputScaling(size_t k, Cell_Frame_HIP* scaling)
{
    if (!mEw || k >= mInputs.size() || !scaling || !scaling->scalingHandle() || mFusedConv)
        return false;
    const int rc = n2d2hip_elemwise_fold_input_scaling(mEw, (int)k, scaling->scalingHandle());
    if (rc == N2D2HIP_ERR_UNSUPPORTED)
        return false;
    checkStatus(rc);
    mFoldedScaling.resize(mInputs.size(), nullptr);
    mFoldedScaling[k] = scaling;
    scaling->setFoldedInto(this);
    return true;
}

bool ElemWiseCell_Frame_HIP::fuseIntoConv(size_t k, Cell_Frame_HIP* conv)
{
    if (!mEw || mInputs.size() != 2 || k > 1 || !conv || !conv->convHandle() || mFusedConv || conv->parentCells().size() != 1)
        return false;
    const int rc = n2d2hip_conv_fuse_sum(conv->convHandle(), mEw, (int)k, sourceOf(mFoldedScaling, mInputs, 1 - k)->desc().dtype);
    if (rc == N2D2HIP_ERR_UNSUPPORTED)
        return false;
    checkStatus(rc);
    mFusedConv = conv;
    mFusedIndex = k;
    conv->setFoldedInto(this);
    return true;
}

bool ElemWiseCell_Frame_HIP::fuseBottleneck(Cell_Frame_HIP* reduce, Cell_Frame_HIP* conv3x3, Cell_Frame_HIP* projection, Cell_Frame_HIP* input)
{
    if (mBottleneck || !mFusedConv || !reduce || !conv3x3 || !input || !reduce->convHandle() || !conv3x3->convHandle()
        || (projection && !projection->convHandle()))
        return false;
    n2d2hip_bottleneck_t b = nullptr;
    const int rc = n2d2hip_bottleneck_create(reduce->convHandle(), conv3x3->convHandle(), mFusedConv->convHandle(),
                                             projection ? projection->convHandle() : nullptr, &b);
    if (rc == N2D2HIP_ERR_UNSUPPORTED)
        return false;
    checkStatus(rc);
    // the library also knows where the one launch is the faster plan
    const n2d2hip_tensor& x = input->getDeviceOutputs().desc();
    if (!n2d2hip_bottleneck_pays(b, x.B, x.H, x.W)) {
        n2d2hip_bottleneck_destroy(b);
        return false;
    }
    mBottleneck = b;
    mBottleneckIn = input;
    mBottleneckCells = {reduce, conv3x3};
    if (projection) mBottleneckCells.push_back(projection);
    for (Cell_Frame_HIP* c : mBottleneckCells)
        c->setFoldedInto(this);
    return true;
}

bool ElemWiseCell_Frame_HIP::fuseChain(Cell_Frame_HIP* conv3x3)
{
    if (mBottleneck || mChainConv || !mFusedConv || !conv3x3 || !conv3x3->convHandle() || conv3x3->foldedInto()
        || conv3x3->parentCells().size() != 1 || !n2d2hip_conv_chain_supported(conv3x3->convHandle(), mFusedConv->convHandle()))
        return false;
    mChainConv = conv3x3;
    conv3x3->setFoldedInto(this);
    return true;
}

void ElemWiseCell_Frame_HIP::clearFusion()
{
    if (mChainConv) {
        mChainConv->setFoldedInto(nullptr);
        mChainConv = nullptr;
    }
    if (mBottleneck) {
        n2d2hip_bottleneck_destroy(mBottleneck);
        mBottleneck = nullptr;
        mBottleneckIn = nullptr;
        for (Cell_Frame_HIP* c : mBottleneckCells)
            c->setFoldedInto(nullptr);
        mBottleneckCells.clear();
    }
    if (mFusedConv) {
        if (mFusedConv->convHandle())
            checkStatus(n2d2hip_conv_fuse_sum(mFusedConv->convHandle(), nullptr, 0, 0));
        mFusedConv->setFoldedInto(nullptr);
        mFusedConv = nullptr;
    }
    for (size_t k = 0; k < mFoldedScaling.size(); ++k) {
        if (!mFoldedScaling[k]) continue;
        if (mEw)
            checkStatus(n2d2hip_elemwise_fold_input_scaling(mEw, (int)k, nullptr));
        mFoldedScaling[k]->setFoldedInto(nullptr);
        mFoldedScaling[k] = nullptr;
    }
}

Registrar<ElemWiseCell> ElemWiseCell_Frame_HIP::mRegistrar("Frame_HIP", ElemWiseCell_Frame_HIP::create, Registrar<ElemWiseCell>::Type<float>());

// ---------------------------------------------------------------- ScalingCell
const char* ScalingCell::Type = "Scaling";

std::pair<double, double> ScalingCell::scalingOutputsRange() const
{
    if (mScaling.getMode() == ScalingMode::NONE)
        throw std::runtime_error("Unsupported scaling mode for cell " + getName() + ".");
    const bool allScalingsPositive = mScaling.allScalingsPositive();
    const double inf = std::numeric_limits<double>::infinity();
    const std::pair<double, double> parents = getOutputsRangeParents();
    if (parents.first >= 0.0 && allScalingsPositive)
        return std::make_pair(0.0, inf);
    return std::make_pair(-inf, inf);
}

template <class T>
ScalingCell_Frame_HIP<T>::ScalingCell_Frame_HIP(const DeepNet& /*deepNet*/, const std::string& name, unsigned int nbOutputs, Scaling scaling)
    : Cell(name, nbOutputs), ScalingCell(std::move(scaling)), mScalingAct(nullptr), mBuiltRevision(~0u), mBuiltUnsigned(-1)
{
}

template <class T>
ScalingCell_Frame_HIP<T>::~ScalingCell_Frame_HIP()
{
    if (mScalingAct) n2d2hip_act_destroy(mScalingAct);
}

template <class T>
void ScalingCell_Frame_HIP<T>::setOutputsDims()
{
    mOutW = mInW;
    mOutH = mInH;
}

template <class T>
void ScalingCell_Frame_HIP<T>::initialize()
{
    if (mInputs.size() != 1)
        throw std::runtime_error("ScalingCell_Frame_HIP " + mName + ": exactly one input is supported");
    if (mScaling.getMode() != ScalingMode::NONE)
        allocateOutputs(&mScaling);
}

template <class T>
void ScalingCell_Frame_HIP<T>::propagate(bool /*inference*/)
{
    prepare();
    launch();
}

template <class T>
void ScalingCell_Frame_HIP<T>::launch()
{
    checkStatus(n2d2hip_scaling_forward(mScalingAct, &mInputs[0]->desc(), &mOutputs.desc(), mStream));
    mOutputs.invalidateHost();
}

template <class T>
bool ScalingCell_Frame_HIP<T>::prepare()
{
    // src/Cell/ScalingCell_Frame.cpp:67-75: mScaling.propagate(*this, in, out, mQuantizedNbBits), no activation
    const bool uns = DeepNetExport::isCellOutputUnsigned(*this);
    bool rebuilt = false;
    if (!mScalingAct || mBuiltRevision != mScalingRevision || mBuiltUnsigned != (int)uns) {
        if (mScalingAct) { n2d2hip_act_destroy(mScalingAct); mScalingAct = nullptr; }
        mScalingAct = makeAct(mScaling, N2D2HIP_ACT_LINEAR, 0.0f, mQuantizedNbBits, uns, mNbOutputs, mName);
        mBuiltRevision = mScalingRevision;
        mBuiltUnsigned = (int)uns;
        if (mOutputs.empty() || mOutputs.desc().dtype != outputDType(&mScaling))
            allocateOutputs(&mScaling);
        rebuilt = true;
    }
    return rebuilt;
}

template <> Registrar<ScalingCell> ScalingCell_Frame_HIP<float>::mRegistrar("Frame_HIP", ScalingCell_Frame_HIP<float>::create,
                                                                            Registrar<ScalingCell>::Type<float>());

// ------------------------------------------------------------------- SGDSolver
SGDSolver::~SGDSolver()
{
    if (mMomentumData) (void)hipFree(mMomentumData);
}

void SGDSolver::setParameter(const std::string& name, double value)
{
    if (name == "LearningRate") mLearningRate = value;
    else if (name == "Momentum") mMomentum = value;
    else if (name == "Decay") mDecay = value;
    else if (name == "IterationSize") mIterationSize = (unsigned int)value;
    else throw std::runtime_error("Parameter does not exist: " + name);
}

double SGDSolver::getLearningRate()
{
    if (mLearningRate == 0.0)
        return 0.0;
    if (mIterationPass < mIterationSize - 1) {
        ++mIterationPass;
        return 0.0;
    }
    mIterationPass = 0;
    ++mNbIterations;
    return mLearningRate;
}

void SGDSolver::update(float& data, float diff, unsigned int batchSize)
{
    // include/Solver/SGDSolver_Frame.hpp:84-109 without momentum / decay: data += rate/(batch*iterSize) * diff,
    // applied on the last pass of an iteration
    const float rate = (float)getLearningRate();
    if (rate == 0.0f)
        return;
    const float rateDiff = rate / ((float)batchSize * (float)mIterationSize);
    data += rateDiff * diff;
}

void SGDSolver::update(float* data, const float* diff, std::size_t n, unsigned int batchSize, void* stream)
{
    const float rate = (float)getLearningRate();
    if (rate == 0.0f)
        return;
    const float rateDiff = rate / ((float)batchSize * (float)mIterationSize);
    const bool plain = (mMomentum == 0.0 && mDecay == 0.0);
    if (!plain && mMomentumSize != n) {
        if (mMomentumData) (void)hipFree(mMomentumData);
        mMomentumData = nullptr;
        checkHip(hipMalloc((void**)&mMomentumData, n * sizeof(float)), "SGDSolver::update()");
        checkHip(hipMemsetAsync(mMomentumData, 0, n * sizeof(float), (hipStream_t)stream), "SGDSolver::update()");
        mMomentumSize = n;
    }
    checkStatus(n2d2hip_sgd_update_f32(data, diff, n, rateDiff, (float)mMomentum, (float)mDecay * rate, plain ? nullptr : mMomentumData,
                                       0, 0.0f, 0.0f, stream));
}

template <> Registrar<SGDSolver> SGDSolver_Frame_HIP<float>::mRegistrar("Frame_HIP", SGDSolver_Frame_HIP<float>::create,
                                                                        Registrar<SGDSolver>::Type<float>());

// ---------------------------------------------------------------- SAT weights
const char* SATQuantizerCell::Type = "SAT";
const char* SATQuantizerActivation::Type = "SAT";
const char* LSQQuantizerCell::Type = "LSQ";
const char* LSQQuantizerActivation::Type = "LSQ";

static float* deviceFloats(size_t n, const char* what)
{
    float* p = nullptr;
    checkHip(hipMalloc((void**)&p, n * sizeof(float)), what);
    return p;
}

static void ensureWorkspace(void*& ws, size_t& bytes, size_t n)
{
    const size_t need = n2d2hip_quantizer_workspace_bytes(n);
    if (bytes >= need) return;
    if (ws) (void)hipFree(ws);
    ws = nullptr;
    checkHip(hipMalloc(&ws, need), "quantizer workspace");
    bytes = need;
}

template <class T>
SATQuantizerCell_Frame_HIP<T>::~SATQuantizerCell_Frame_HIP()
{
    for (auto& b : mW) { (void)hipFree(b.q); (void)hipFree(b.diffFp); }
    if (mStats) (void)hipFree(mStats);
    if (mWorkspace) (void)hipFree(mWorkspace);
}

template <class T>
void SATQuantizerCell_Frame_HIP<T>::addWeights(float* weights, float* diffQuantizedWeights, std::size_t size, std::size_t outputsSize)
{
    QuantizerBuffers b;
    b.fp = weights; b.diffQ = diffQuantizedWeights; b.size = size; b.outputsSize = outputsSize;
    b.q = deviceFloats(size, "SATQuantizerCell_Frame_HIP::addWeights()");
    b.diffFp = deviceFloats(size, "SATQuantizerCell_Frame_HIP::addWeights()");
    mW.push_back(b);
    mOutputsSize += outputsSize;       // SATQuantizerCell_Frame.cpp:79: sum of dimB*dimY*dimX over the weight tensors
}

template <class T>
int SATQuantizerCell_Frame_HIP<T>::satMode() const
{
    // SATQuantizerCell_Frame.cpp:188-200
    if (mQuantMode == QuantizerCell::FullRange) return mApplyQuantization ? N2D2HIP_SAT_FULLRANGE : N2D2HIP_SAT_NONE;
    if (mQuantMode == QuantizerCell::Symmetric) return mApplyQuantization ? N2D2HIP_SAT_SYMRANGE : N2D2HIP_SAT_NONE;
    if (mQuantMode == QuantizerCell::Asymmetric) return mApplyQuantization ? N2D2HIP_SAT_ASYMRANGE : N2D2HIP_SAT_NONE_ASYM;
    return mApplyQuantization ? N2D2HIP_SAT_DEFAULT : N2D2HIP_SAT_NONE;
}

template <class T>
void SATQuantizerCell_Frame_HIP<T>::initialize()
{
    if (!mStats && !mW.empty())
        mStats = deviceFloats(2 * mW.size(), "SATQuantizerCell_Frame_HIP::initialize()");
    propagate();         // initializeQWeights
}

template <class T>
void SATQuantizerCell_Frame_HIP<T>::propagate()
{
    if (!mStats && !mW.empty())
        mStats = deviceFloats(2 * mW.size(), "SATQuantizerCell_Frame_HIP::propagate()");
    for (size_t k = 0; k < mW.size(); ++k) {
        ensureWorkspace(mWorkspace, mWorkspaceBytes, mW[k].size);
        checkStatus(n2d2hip_sat_weight_forward(mW[k].fp, mW[k].q, mW[k].size, (float)mRange, satMode(), mApplyScaling ? 1 : 0,
                                               (unsigned)mOutputsSize, mStats + 2 * k, mWorkspace, mWorkspaceBytes, mStream));
    }
}

template <class T>
void SATQuantizerCell_Frame_HIP<T>::back_propagate()
{
    for (size_t k = 0; k < mW.size(); ++k) {
        // SATQuantizerCell_Frame.cpp:249-283: Asymmetric and FullRange select their kernel by QuantMode alone
        int mode = N2D2HIP_SAT_DEFAULT;
        if (mQuantMode == QuantizerCell::Asymmetric) mode = N2D2HIP_SAT_ASYMRANGE;
        else if (mQuantMode == QuantizerCell::FullRange) mode = N2D2HIP_SAT_FULLRANGE;
        checkStatus(n2d2hip_sat_weight_backward(mW[k].diffQ, mW[k].fp, mW[k].diffFp, mW[k].size, (float)mRange, mode, mApplyScaling ? 1 : 0,
                                                mStats + 2 * k, mStream));
    }
}

template <class T>
std::pair<float, float> SATQuantizerCell_Frame_HIP<T>::getStats(unsigned int k) const
{
    float h[2] = {0, 0};
    checkHip(hipMemcpy(h, mStats + 2 * k, sizeof(h), hipMemcpyDeviceToHost), "SATQuantizerCell_Frame_HIP::getStats()");
    return std::make_pair(h[0], h[1]);
}

template <> Registrar<SATQuantizerCell> SATQuantizerCell_Frame_HIP<float>::mRegistrar("Frame_HIP", SATQuantizerCell_Frame_HIP<float>::create,
                                                                                      Registrar<SATQuantizerCell>::Type<float>());

// ------------------------------------------------------------ SAT activations
template <class T>
SATQuantizerActivation_Frame_HIP<T>::~SATQuantizerActivation_Frame_HIP()
{
    if (mDev) (void)hipFree(mDev);
    if (mFp) (void)hipFree(mFp);
    if (mWorkspace) (void)hipFree(mWorkspace);
}

template <class T>
void SATQuantizerActivation_Frame_HIP<T>::lazyInit(std::size_t size, bool needCopy)
{
    if (!mDev) {
        // alpha tensor {1,1,1,1} initialised from the Alpha parameter at the first propagate
        mDev = deviceFloats(2, "SATQuantizerActivation_Frame_HIP");
        const float h[2] = {(float)mAlphaParameter, 0.0f};
        checkHip(hipMemcpy(mDev, h, sizeof(h), hipMemcpyHostToDevice), "SATQuantizerActivation_Frame_HIP");
    }
    if (needCopy && mFpSize != size) {
        if (mFp) (void)hipFree(mFp);
        mFp = deviceFloats(size, "SATQuantizerActivation_Frame_HIP");
        mFpSize = size;
    }
}

template <class T>
void SATQuantizerActivation_Frame_HIP<T>::propagate(float* inOut, std::size_t size, bool inference)
{
    lazyInit(size, !inference);
    checkStatus(n2d2hip_sat_act_forward(inOut, inference ? nullptr : mFp, size, (float)mRange, mDev, mStream));
}

template <class T>
void SATQuantizerActivation_Frame_HIP<T>::back_propagate(const float* diffInput, float* diffOutput, std::size_t size)
{
    if (!mFp || mFpSize != size)
        throw std::runtime_error("SATQuantizerActivation_Frame_HIP::back_propagate(): no full-precision activations saved (propagate with inference = false first)");
    lazyInit(size, true);
    ensureWorkspace(mWorkspace, mWorkspaceBytes, size);
    const float beta = (mSolver && !mSolver->isNewIteration()) ? 1.0f : 0.0f;
    checkStatus(n2d2hip_sat_act_backward(diffInput, mFp, diffOutput, size, (float)mRange, mDev, beta, mDev + 1, mWorkspace, mWorkspaceBytes, mStream));
}

template <class T>
float SATQuantizerActivation_Frame_HIP<T>::getAlpha()
{
    lazyInit(0, false);
    float h = 0;
    checkHip(hipMemcpy(&h, mDev, sizeof(float), hipMemcpyDeviceToHost), "getAlpha");
    return h;
}
template <class T>
float SATQuantizerActivation_Frame_HIP<T>::getDiffAlpha()
{
    lazyInit(0, false);
    float h = 0;
    checkHip(hipMemcpy(&h, mDev + 1, sizeof(float), hipMemcpyDeviceToHost), "getDiffAlpha");
    return h;
}
template <class T>
void SATQuantizerActivation_Frame_HIP<T>::update(unsigned int batchSize)
{
    if (!mSolver) return;
    lazyInit(0, false);
    mSolver->update(mDev, mDev + 1, 1, batchSize, mStream);       // alpha and its gradient stay on the device
}

template <> Registrar<SATQuantizerActivation> SATQuantizerActivation_Frame_HIP<float>::mRegistrar(
    "Frame_HIP", SATQuantizerActivation_Frame_HIP<float>::create, Registrar<SATQuantizerActivation>::Type<float>());

// ---------------------------------------------------------------- LSQ weights
template <class T>
LSQQuantizerCell_Frame_HIP<T>::~LSQQuantizerCell_Frame_HIP()
{
    for (auto& b : mW) { (void)hipFree(b.q); (void)hipFree(b.diffFp); }
    if (mDev) (void)hipFree(mDev);
    if (mWorkspace) (void)hipFree(mWorkspace);
}

template <class T>
void LSQQuantizerCell_Frame_HIP<T>::addWeights(float* weights, float* diffQuantizedWeights, std::size_t size, std::size_t outputsSize)
{
    QuantizerBuffers b;
    b.fp = weights; b.diffQ = diffQuantizedWeights; b.size = size; b.outputsSize = outputsSize;
    b.q = deviceFloats(size, "LSQQuantizerCell_Frame_HIP::addWeights()");
    b.diffFp = deviceFloats(size, "LSQQuantizerCell_Frame_HIP::addWeights()");
    mW.push_back(b);
}

// mean(|w|) of a device tensor, for the step-size initialisation of the LSQ paper
static double meanAbsOnHost(const float* dev, size_t n)
{
    std::vector<float> h(n);
    checkHip(hipMemcpy(h.data(), dev, n * sizeof(float), hipMemcpyDeviceToHost), "LSQ step-size initialisation");
    double s = 0.0;
    for (float v : h) s += std::fabs((double)v);
    return s / (double)n;
}

template <class T>
void LSQQuantizerCell_Frame_HIP<T>::initialize()
{
    // LSQQuantizerCell_Frame.cpp:106-145: range [-(R+1)/2, (R-1)/2]; optimal initial step 2*mean|w|/sqrt(hi)
    mLo = -(int)((mRange + 1) >> 1);
    mHi = (int)((mRange - 1) >> 1);
    size_t total = 0;
    for (auto& b : mW) total += b.size;
    if (!mDev) {
        if (mSetOptInitStepSize && !mW.empty())
            mStepSizeVal = 2.0f * (float)(meanAbsOnHost(mW[0].fp, mW[0].size) / std::sqrt((double)mHi));
        mDev = deviceFloats(2, "LSQQuantizerCell_Frame_HIP::initialize()");
        const float h[2] = {mStepSizeVal, 0.0f};
        checkHip(hipMemcpy(mDev, h, sizeof(h), hipMemcpyHostToDevice), "LSQQuantizerCell_Frame_HIP::initialize()");
    }
    mGradScale = (float)(1.0 / std::sqrt((double)total * (double)mHi));
    mInitialized = true;
    propagate();
}

template <class T>
void LSQQuantizerCell_Frame_HIP<T>::propagate()
{
    if (!mInitialized) { initialize(); return; }
    for (auto& b : mW)
        checkStatus(n2d2hip_lsq_forward(b.fp, b.q, b.size, mDev, mLo, mHi, nullptr));
}

template <class T>
void LSQQuantizerCell_Frame_HIP<T>::back_propagate()
{
    if (!mInitialized)
        throw std::runtime_error("LSQQuantizerCell_Frame_HIP::back_propagate(): not initialized");
    // the step-size gradient accumulates over the weight tensors of the cell and, inside one solver
    // iteration, over passes; the scale factor is applied once per call as the reference does
    float beta = (mSolver && !mSolver->isNewIteration()) ? 1.0f : 0.0f;
    for (size_t k = 0; k < mW.size(); ++k) {
        ensureWorkspace(mWorkspace, mWorkspaceBytes, mW[k].size);
        const bool last = k + 1 == mW.size();
        checkStatus(n2d2hip_lsq_backward(mW[k].diffQ, mW[k].fp, mW[k].diffFp, mW[k].size, mDev, mLo, mHi, last ? mGradScale : 1.0f, beta,
                                         mDev + 1, mWorkspace, mWorkspaceBytes, nullptr));
        beta = 1.0f;
    }
}

template <class T>
float LSQQuantizerCell_Frame_HIP<T>::getStepSize()
{
    float h = 0;
    checkHip(hipMemcpy(&h, mDev, sizeof(float), hipMemcpyDeviceToHost), "getStepSize");
    return h;
}
template <class T>
float LSQQuantizerCell_Frame_HIP<T>::getDiffStepSize()
{
    float h = 0;
    checkHip(hipMemcpy(&h, mDev + 1, sizeof(float), hipMemcpyDeviceToHost), "getDiffStepSize");
    return h;
}
template <class T>
void LSQQuantizerCell_Frame_HIP<T>::update(unsigned int batchSize)
{
    if (!mSolver) return;
    float h[2];
    checkHip(hipMemcpy(h, mDev, sizeof(h), hipMemcpyDeviceToHost), "LSQQuantizerCell_Frame_HIP::update()");
    mSolver->update(h[0], h[1], batchSize);
    checkHip(hipMemcpy(mDev, h, sizeof(float), hipMemcpyHostToDevice), "LSQQuantizerCell_Frame_HIP::update()");
}

template <> Registrar<LSQQuantizerCell> LSQQuantizerCell_Frame_HIP<float>::mRegistrar("Frame_HIP", LSQQuantizerCell_Frame_HIP<float>::create,
                                                                                      Registrar<LSQQuantizerCell>::Type<float>());

// ------------------------------------------------------------ LSQ activations
template <class T>
LSQQuantizerActivation_Frame_HIP<T>::~LSQQuantizerActivation_Frame_HIP()
{
    if (mDev) (void)hipFree(mDev);
    if (mFp) (void)hipFree(mFp);
    if (mWorkspace) (void)hipFree(mWorkspace);
}

template <class T>
void LSQQuantizerActivation_Frame_HIP<T>::propagate(float* inOut, std::size_t size, bool /*inference*/)
{
    // LSQQuantizerActivation_Frame.cpp:92-141: range [0, R]; the full-precision input is always saved
    mGradScale = (float)(1.0 / std::sqrt((double)size * (double)mRange));
    if (!mDev) {
        if (mSetOptInitStepSize) {
            std::vector<float> h(size);
            checkHip(hipMemcpy(h.data(), inOut, size * sizeof(float), hipMemcpyDeviceToHost), "LSQ activation step-size initialisation");
            double s = 0.0;
            for (float v : h) s += std::fabs((double)v);
            mStepSizeParameter = 2.0f * (float)((s / (double)size) / std::sqrt((double)mRange));
            mSetOptInitStepSize = false;
        }
        mDev = deviceFloats(2, "LSQQuantizerActivation_Frame_HIP");
        const float h2[2] = {mStepSizeParameter, 0.0f};
        checkHip(hipMemcpy(mDev, h2, sizeof(h2), hipMemcpyHostToDevice), "LSQQuantizerActivation_Frame_HIP");
    }
    if (mFpSize != size) {
        if (mFp) (void)hipFree(mFp);
        mFp = deviceFloats(size, "LSQQuantizerActivation_Frame_HIP");
        mFpSize = size;
    }
    checkHip(hipMemcpyAsync(mFp, inOut, size * sizeof(float), hipMemcpyDeviceToDevice, nullptr), "LSQQuantizerActivation_Frame_HIP::propagate()");
    checkStatus(n2d2hip_lsq_forward(mFp, inOut, size, mDev, 0, (int)mRange, nullptr));
}

template <class T>
void LSQQuantizerActivation_Frame_HIP<T>::back_propagate(const float* diffInput, float* diffOutput, std::size_t size)
{
    if (!mDev || !mFp || mFpSize != size)
        throw std::runtime_error("LSQQuantizerActivation_Frame_HIP::back_propagate(): propagate first");
    ensureWorkspace(mWorkspace, mWorkspaceBytes, size);
    const float beta = (mSolver && !mSolver->isNewIteration()) ? 1.0f : 0.0f;
    checkStatus(n2d2hip_lsq_backward(diffInput, mFp, diffOutput, size, mDev, 0, (int)mRange, mGradScale, beta, mDev + 1, mWorkspace,
                                     mWorkspaceBytes, nullptr));
}

template <class T>
float LSQQuantizerActivation_Frame_HIP<T>::getStepSize()
{
    float h = 0;
    checkHip(hipMemcpy(&h, mDev, sizeof(float), hipMemcpyDeviceToHost), "getStepSize");
    return h;
}
template <class T>
float LSQQuantizerActivation_Frame_HIP<T>::getDiffStepSize()
{
    float h = 0;
    checkHip(hipMemcpy(&h, mDev + 1, sizeof(float), hipMemcpyDeviceToHost), "getDiffStepSize");
    return h;
}
template <class T>
void LSQQuantizerActivation_Frame_HIP<T>::update(unsigned int batchSize)
{
    if (!mSolver || !mDev) return;
    float h[2];
    checkHip(hipMemcpy(h, mDev, sizeof(h), hipMemcpyDeviceToHost), "LSQQuantizerActivation_Frame_HIP::update()");
    mSolver->update(h[0], h[1], batchSize);
    checkHip(hipMemcpy(mDev, h, sizeof(float), hipMemcpyHostToDevice), "LSQQuantizerActivation_Frame_HIP::update()");
}

template <> Registrar<LSQQuantizerActivation> LSQQuantizerActivation_Frame_HIP<float>::mRegistrar(
    "Frame_HIP", LSQQuantizerActivation_Frame_HIP<float>::create, Registrar<LSQQuantizerActivation>::Type<float>());

template class SATQuantizerCell_Frame_HIP<float>;
template class SATQuantizerActivation_Frame_HIP<float>;
template class LSQQuantizerCell_Frame_HIP<float>;
template class LSQQuantizerActivation_Frame_HIP<float>;
template class ConvCell_Frame_HIP<float>;
template class FcCell_Frame_HIP<float>;
template class PoolCell_Frame_HIP<float>;
template class ScalingCell_Frame_HIP<float>;

// -------------------------------------------------------------------- DeepNet
void DeepNet::addCell(const std::shared_ptr<Cell>& cell, const std::vector<std::shared_ptr<Cell> >& parents)
{
    if (mCells.count(cell->getName()))
        throw std::runtime_error("DeepNet::addCell(): cell " + cell->getName() + " already exists");
    auto frame = std::dynamic_pointer_cast<Cell_Frame_HIP>(cell);
    if (!frame)
        throw std::runtime_error("DeepNet::addCell(): cell " + cell->getName() + " is not a Frame_HIP cell");
    if (parents.empty()) {
        if (mEnvB == 0)
            throw std::runtime_error("DeepNet::addCell(): set the stimuli size before connecting cell " + cell->getName() + " to the environment");
        frame->addInput(mStimuli, mEnvC, mEnvH, mEnvW, mEnvB);
    }
    for (const auto& p : parents) {
        auto pf = std::dynamic_pointer_cast<Cell_Frame_HIP>(p);
        if (!pf)
            throw std::runtime_error("DeepNet::addCell(): parent of " + cell->getName() + " is not a Frame_HIP cell");
        frame->addInput(pf.get());
    }
    mOrder.push_back(cell);
    mFrames.push_back(frame.get());
    mCells[cell->getName()] = cell;
    mPlanned = false;
}

std::shared_ptr<Cell> DeepNet::getCell(const std::string& name) const
{
    auto it = mCells.find(name);
    if (it == mCells.end())
        throw std::runtime_error("DeepNet::getCell(): layer " + name + " does not exist");
    return it->second;
}

void DeepNet::setStimuli(unsigned int nbChannels, unsigned int height, unsigned int width, unsigned int batchSize)
{
    mEnvC = nbChannels; mEnvH = height; mEnvW = width; mEnvB = batchSize;
}

void DeepNet::setStimuliData(const Tensor<Float_T>& data)
{
    // network input unsigned <=> DeepNetExport::mEnvDataUnsigned (StimuliProviderExport::unsignedStimuli)
    const int dtype = (CellExport::mPrecision > 0 && DeepNetExport::mUnsignedData && DeepNetExport::mEnvDataUnsigned) ? N2D2HIP_U8B : N2D2HIP_I8;
    if (mStimuli.empty() || mStimuli.desc().dtype != dtype)
        mStimuli.resize((int)mEnvB, (int)mEnvC, (int)mEnvH, (int)mEnvW, dtype, 0, true);
    for (size_t i = 0; i < data.size(); ++i)
        toInteger(data(i), dtype == N2D2HIP_U8B ? 0 : -128, dtype == N2D2HIP_U8B ? 255 : 127, "stimuli");
    mStimuliHost = data;          // (the fusion plan may change the stimuli's layout on the device: they are converted again then)
    mStimuli.synchronizeHToD(data);
}

// The stimuli go to the device space-to-depth when the one cell reading them is a first-layer convolution the device
// library serves that way (n2d2hip_conv_s2d_halo), with the max pooling that convolution computes, if it does; otherwise
// as plain NHWC pixels.  Called by planFusion(), behind the decision about that pooling.
void DeepNet::layoutStimuli()
{
    if (mStimuli.empty())
        return;
    Cell_Frame_HIP* reader = nullptr;
    size_t readers = 0;
    for (Cell_Frame_HIP* f : mFrames)
        for (size_t k = 0; k < f->nbInputs(); ++k)
            if (f->inputTensor(k) == &mStimuli) { reader = f; ++readers; }
    int halo = -1;
    if (mFusion && readers == 1 && reader->convHandle() && reader->nbInputs() == 1) {
        const n2d2hip_pool_desc* pd = nullptr;
        n2d2hip_pool_desc d;
        if (auto* pool = dynamic_cast<PoolCell_Frame_HIP<float>*>(reader->foldedInto())) {
            d = pool->poolDescriptor();
            pd = &d;
        }
        if (!reader->foldedInto() || pd)
            halo = n2d2hip_conv_s2d_halo(reader->convHandle(), pd, (int)mEnvH, (int)mEnvW);
    }
    const n2d2hip_tensor& now = mStimuli.desc();
    const bool wantS2d = halo >= 0;
    if (wantS2d == (now.layout == N2D2HIP_S2D) && (!wantS2d || now.halo == halo))
        return;
    if (wantS2d)
        mStimuli.resizeSpaceToDepth((int)mEnvB, (int)mEnvC, (int)mEnvH, (int)mEnvW, now.dtype, halo);
    else
        mStimuli.resize((int)mEnvB, (int)mEnvC, (int)mEnvH, (int)mEnvW, now.dtype, 0, true);
    if (!mStimuliHost.empty())
        mStimuli.synchronizeHToD(mStimuliHost);
}

void DeepNet::initialize()
{
    const int dtype = (CellExport::mPrecision > 0 && DeepNetExport::mUnsignedData && DeepNetExport::mEnvDataUnsigned) ? N2D2HIP_U8B : N2D2HIP_I8;
    if (mEnvB > 0 && mStimuli.empty())
        mStimuli.resize((int)mEnvB, (int)mEnvC, (int)mEnvH, (int)mEnvW, dtype, 0, true);
    for (auto& c : mOrder)
        std::dynamic_pointer_cast<Cell_Frame_HIP>(c)->initialize();
}

void DeepNet::propagate(bool /*inference*/)
{
    bool rebuilt = false;
    for (Cell_Frame_HIP* f : mFrames)
        rebuilt = f->prepare() || rebuilt;
    if (rebuilt || !mPlanned) {
        if (mFusion) {
            planFusion();
        } else {
            layoutStimuli();
            mPlanned = true;
        }
    }
    for (Cell_Frame_HIP* f : mFrames) {
        if (!f->foldedInto())
            f->launch();
    }
}

void DeepNet::setFusion(bool enabled)
{
    if (!enabled) {
        for (Cell_Frame_HIP* f : mFrames) {
            if (auto* ew = dynamic_cast<ElemWiseCell_Frame_HIP*>(f))
                ew->clearFusion();
            if (auto* pool = dynamic_cast<PoolCell_Frame_HIP<float>*>(f))
                pool->clearFusion();
            if (auto* conv = dynamic_cast<ConvCell_Frame_HIP<float>*>(f))
                conv->clearFusion();
            if (auto* fc = dynamic_cast<FcCell_Frame_HIP<float>*>(f))
                fc->clearFusion();
            f->setOutputsHalo(0);
        }
    }
    mFusion = enabled;
    mPlanned = false;
}

size_t DeepNet::nbFoldedCells() const
{
    return (size_t)std::count_if(mFrames.begin(), mFrames.end(), [](const Cell_Frame_HIP* f) { return f->foldedInto() != nullptr; });
}

// Every handle is current when this runs (all cells prepared).  Decisions follow the graph only; the device library has
// the last word on each candidate and the cells stay separate launches where it declines.
void DeepNet::planFusion()
{
    std::map<const Cell_Frame_HIP*, int> consumers, order;
    order[nullptr] = -1;
    for (size_t i = 0; i < mFrames.size(); ++i) {
        order[mFrames[i]] = (int)i;
        for (Cell_Frame_HIP* p : mFrames[i]->parentCells())
            ++consumers[p];
    }
    // a max pooling that is the only reader of a first-layer convolution is computed by that convolution's launch
    for (Cell_Frame_HIP* f : mFrames) {
        auto* pool = dynamic_cast<PoolCell_Frame_HIP<float>*>(f);
        if (!pool) continue;
        pool->clearFusion();
        const std::vector<Cell_Frame_HIP*>& parents = pool->parentCells();
        if (parents.size() == 1 && parents[0] && consumers[parents[0]] == 1)
            pool->fuseFirstConv(parents[0]);
    }
    layoutStimuli();
    // a 1x1 convolution that is the only reader of a 3x3 depthwise convolution computes it in its own launch
    for (Cell_Frame_HIP* f : mFrames) {
        auto* conv = dynamic_cast<ConvCell_Frame_HIP<float>*>(f);
        if (!conv) continue;
        conv->clearFusion();
        const std::vector<Cell_Frame_HIP*>& parents = conv->parentCells();
        if (parents.size() == 1 && parents[0] && consumers[parents[0]] == 1)
            conv->fuseDepthwise(parents[0]);
    }
    for (Cell_Frame_HIP* f : mFrames) {
        auto* ew = dynamic_cast<ElemWiseCell_Frame_HIP*>(f);
        if (!ew) continue;
        ew->clearFusion();
        const std::vector<Cell_Frame_HIP*>& parents = ew->parentCells();
        // one ScalingCell read by this sum alone is applied inside the sum
        size_t scaled = parents.size();
        for (size_t k = 0; k < parents.size() && scaled == parents.size(); ++k) {
            if (parents[k] && parents[k]->scalingHandle() && consumers[parents[k]] == 1 && !parents[k]->foldedInto()
                && ew->foldInputScaling(k, parents[k]))
                scaled = k;
        }
        if (parents.size() != 2) continue;
        // the convolution that runs last among the two producers takes the sum into its epilogue
        for (size_t k : {(size_t)1, (size_t)0}) {
            Cell_Frame_HIP* conv = parents[k];
            if (!conv || !conv->convHandle() || consumers[conv] != 1 || conv->foldedInto() || scaled == k)
                continue;
            const Cell_Frame_HIP* other = scaled == 1 - k ? parents[1 - k]->parentCells().at(0) : parents[1 - k];
            if (other == conv || order[other] > order[conv])
                continue;
            if (ew->fuseIntoConv(k, conv))
                break;
        }
    }
    // A residual block with a projection shortcut, reduce (1x1) -> 3x3 -> expand (1x1) + projection (1x1) + sum, runs as one
    // launch where the device library takes it.  The sum sits in the convolution that runs last, which is the projection
    // when the graph lists it behind the main branch: it is moved into the expansion first (and back if the library
    // declines).  The block's input then carries a border of one pixel, which its producer must be able to write.
    std::map<const Cell_Frame_HIP*, bool> bottleneckInput;
    for (Cell_Frame_HIP* f : mFrames) {
        auto* ew = dynamic_cast<ElemWiseCell_Frame_HIP*>(f);
        if (!ew || !ew->fusedConv() || ew->parentCells().size() != 2)
            continue;
        const size_t k = ew->fusedIndex();
        Cell_Frame_HIP* holder = ew->fusedConv();
        Cell_Frame_HIP* other = ew->parentCells()[1 - k];
        if (!other || !other->convHandle() || ew->hasFoldedScaling(1 - k) || consumers[other] != 1 || other->foldedInto())
            continue;
        auto single_conv_parent = [&](Cell_Frame_HIP* c) -> Cell_Frame_HIP* {
            const std::vector<Cell_Frame_HIP*>& ps = c->parentCells();
            return ps.size() == 1 && ps[0] && ps[0]->convHandle() ? ps[0] : nullptr;
        };
        // which of the two convolutions ends the main branch (its input is a convolution whose input is a convolution)?
        Cell_Frame_HIP* expand = nullptr;
        Cell_Frame_HIP* proj = nullptr;
        for (Cell_Frame_HIP* cand : {holder, other}) {
            Cell_Frame_HIP* b3 = single_conv_parent(cand);
            if (b3 && single_conv_parent(b3)) { expand = cand; proj = cand == holder ? other : holder; break; }
        }
        if (!expand)
            continue;
        Cell_Frame_HIP* conv3 = single_conv_parent(expand);
        Cell_Frame_HIP* reduce = single_conv_parent(conv3);
        if (reduce->parentCells().size() != 1 || proj->parentCells().size() != 1)
            continue;
        Cell_Frame_HIP* x = reduce->parentCells()[0];
        if (!x || proj->parentCells()[0] != x || consumers[x] != 2 || consumers[reduce] != 1 || consumers[conv3] != 1
            || reduce->foldedInto() || conv3->foldedInto())
            continue;
        auto* xpool = dynamic_cast<PoolCell_Frame_HIP<float>*>(x);
        auto* xsum = dynamic_cast<ElemWiseCell_Frame_HIP*>(x);
        if (!((xpool && xpool->writesHalo()) || (xsum && xsum->fusedConv())))
            continue;
        const size_t kExpand = expand == holder ? k : 1 - k;
        if (expand != holder) {
            ew->clearFusion();
            if (!ew->fuseIntoConv(kExpand, expand)) {
                ew->fuseIntoConv(k, holder);
                continue;
            }
        }
        if (ew->fuseBottleneck(reduce, conv3, proj, x)) {
            bottleneckInput[x] = true;
        } else if (expand != holder) {
            ew->clearFusion();
            ew->fuseIntoConv(k, holder);
        }
    }
    // An output that only convolutions read carries the largest padding among them as a border of zeros, when all of them
    // run on the kernel that takes such tensors and the launch that produces it can write one: a convolution of that kind,
    // a sum computed in a convolution's epilogue, a 2x2 / 3x3 max pooling.  A sum of that kind may also read such a
    // tensor as its other input (the epilogue finds the pixels past their borders): ResNet-18's block inputs.
    std::map<const Cell_Frame_HIP*, int> halo;
    std::map<const Cell_Frame_HIP*, bool> refused;
    for (Cell_Frame_HIP* f : mFrames) {
        auto* ew = dynamic_cast<ElemWiseCell_Frame_HIP*>(f);
        const std::vector<Cell_Frame_HIP*>& parents = f->parentCells();
        for (size_t k = 0; k < parents.size(); ++k) {
            Cell_Frame_HIP* p = parents[k];
            if (!p) continue;
            if (f->convHandle() && parents.size() == 1 && n2d2hip_conv_accepts_halo(f->convHandle()))
                halo[p] = std::max(halo[p], f->maxPadding());
            else if (ew && ew->fusedConv() && k != ew->fusedIndex() && !ew->hasFoldedScaling(k))
                continue;
            else
                refused[p] = true;
        }
    }
    for (Cell_Frame_HIP* f : mFrames) {
        auto* conv = dynamic_cast<ConvCell_Frame_HIP<float>*>(f);
        auto* ew = dynamic_cast<ElemWiseCell_Frame_HIP*>(f);
        auto* pool = dynamic_cast<PoolCell_Frame_HIP<float>*>(f);
        const bool writes = (f->convHandle() && !f->foldedInto() && n2d2hip_conv_accepts_halo(f->convHandle())
                             && !(conv && conv->computesDepthwise()))
            || (ew && ew->fusedConv()) || (pool && pool->writesHalo());
        halo[f] = bottleneckInput[f] ? 1 : (writes && !refused[f] ? halo[f] : 0);
        f->setOutputsHalo(halo[f]);
    }
    // In the other residual blocks the 3x3 convolution, whose output only the expansion that holds the sum reads, runs in
    // that launch, where the device library takes the pair and the 3x3 convolution's input carries its padding.
    for (Cell_Frame_HIP* f : mFrames) {
        auto* ew = dynamic_cast<ElemWiseCell_Frame_HIP*>(f);
        if (!ew || !ew->fusedConv() || ew->bottleneckInput())
            continue;
        const std::vector<Cell_Frame_HIP*>& ps = ew->fusedConv()->parentCells();
        Cell_Frame_HIP* conv3 = ps.size() == 1 ? ps[0] : nullptr;
        if (!conv3 || !conv3->convHandle() || consumers[conv3] != 1 || conv3->parentCells().size() != 1 || !conv3->parentCells()[0]
            || halo[conv3->parentCells()[0]] < 1)
            continue;
        ew->fuseChain(conv3);
    }
    // Fully-connected cells in a row, each read by the next alone (a classifier head), run in the launch of the last one,
    // up to three of them, where the device library takes the run.
    std::map<const Cell_Frame_HIP*, Cell_Frame_HIP*> reader;
    for (Cell_Frame_HIP* f : mFrames) {
        if (auto* fc = dynamic_cast<FcCell_Frame_HIP<float>*>(f))
            fc->clearFusion();
        for (Cell_Frame_HIP* p : f->parentCells())
            reader[p] = f;
    }
    auto feedsOneFc = [&](Cell_Frame_HIP* c) {
        auto* next = consumers[c] == 1 ? dynamic_cast<FcCell_Frame_HIP<float>*>(reader[c]) : nullptr;
        return next && next->parentCells().size() == 1;
    };
    for (Cell_Frame_HIP* f : mFrames) {
        auto* last = dynamic_cast<FcCell_Frame_HIP<float>*>(f);
        if (!last || last->parentCells().size() != 1 || feedsOneFc(last))
            continue;
        std::vector<FcCell_Frame_HIP<float>*> earlier;
        for (Cell_Frame_HIP* c = last; earlier.size() < 2;) {
            auto* p = dynamic_cast<FcCell_Frame_HIP<float>*>(c->parentCells()[0]);
            if (!p || consumers[p] != 1 || p->parentCells().size() != 1 || p->foldedInto())
                break;
            earlier.insert(earlier.begin(), p);
            c = p;
        }
        // the library may take the last two cells where it declines all three
        while (!earlier.empty() && !last->fuseChain(earlier))
            earlier.erase(earlier.begin());
    }
    mPlanned = true;
}

void DeepNet::synchronize()
{
    checkHip(hipDeviceSynchronize(), "DeepNet::synchronize()");
}

// ------------------------------------------------------------------ INI subset
namespace {
std::string trim(const std::string& s)
{
    const size_t a = s.find_first_not_of(" \t\r\n");
    if (a == std::string::npos) return "";
    const size_t b = s.find_last_not_of(" \t\r\n");
    return s.substr(a, b - a + 1);
}
std::vector<std::string> split(const std::string& s, const std::string& seps)
{
    std::vector<std::string> out;
    size_t pos = 0;
    while (pos <= s.size()) {
        const size_t next = s.find_first_of(seps, pos);
        const std::string tok = trim(s.substr(pos, next == std::string::npos ? std::string::npos : next - pos));
        if (!tok.empty()) out.push_back(tok);
        if (next == std::string::npos) break;
        pos = next + 1;
    }
    return out;
}
typedef std::map<std::string, std::string> Section;
unsigned int getUInt(const Section& s, const std::string& key, unsigned int def, bool required = false, const std::string& sec = "")
{
    auto it = s.find(key);
    if (it == s.end()) {
        if (required) throw std::runtime_error("Missing parameter " + key + " in section [" + sec + "]");
        return def;
    }
    return (unsigned int)std::stoul(it->second);
}
std::vector<unsigned int> getDims(const Section& s, const std::string& vec, const std::string& scalar, const std::string& x, const std::string& y,
                                  unsigned int def)
{
    auto it = s.find(vec);
    if (it != s.end()) {
        std::vector<unsigned int> v;
        for (const auto& t : split(it->second, " \t")) v.push_back((unsigned int)std::stoul(t));
        if (v.size() == 1) v.push_back(v[0]);
        return v;
    }
    const unsigned int both = getUInt(s, scalar, def);
    return {getUInt(s, x, both), getUInt(s, y, both)};
}
// The connection map between one parent and a cell, {nbOutputs, nbChannels}, from the section's Mapping keys
// (src/Generator/MappingGenerator.cpp:33-201): equal groups (Mapping.NbGroups / Mapping.ChannelsPerGroup), a matrix written
// out (Mapping(parent)= one row per channel), a patch stepped along the diagonal (Mapping.Size / Stride / Offset /
// NbIterations, each also as Mapping(parent).Key for one parent), every connection when the section has none of them.
Tensor<bool> generateMapping(const Section& s, const std::string& section, const std::string& parentName, std::size_t nbOutputs,
                             std::size_t nbChannels)
{
    const std::string own = "Mapping(" + parentName + ")";
    const bool byGroups = s.count("Mapping.NbGroups") != 0, byWidth = s.count("Mapping.ChannelsPerGroup") != 0;
    if (byGroups && byWidth)
        throw std::runtime_error("Mapping.NbGroups and Mapping.ChannelsPerGroup are mutually exclusive in section [" + section + "]");
    if (byGroups || byWidth) {
        const std::size_t given = getUInt(s, byGroups ? "Mapping.NbGroups" : "Mapping.ChannelsPerGroup", 0);
        if (given == 0 || given > nbChannels)
            throw std::runtime_error("Mapping.NbGroups must be a multiple of the number of input channels in section [" + section + "]");
        const std::size_t groups = byGroups ? given : nbChannels / given, width = byGroups ? nbChannels / given : given;
        if (nbChannels % groups != 0)
            throw std::runtime_error("Mapping.NbGroups must be a multiple of the number of input channels in section [" + section + "]");
        Tensor<bool> map({nbOutputs, nbChannels}, false);
        std::size_t firstOutput = 0;
        for (std::size_t g = 0; g < groups; ++g) {
            const std::size_t outputsHere = (nbOutputs - firstOutput) / (groups - g);     // the outputs left, shared out evenly
            for (std::size_t o = firstOutput; o < firstOutput + outputsHere; ++o)
                for (std::size_t ch = g * width; ch < (g + 1) * width; ++ch)
                    map.set(o, ch, true);
            firstOutput += outputsHere;
        }
        return map;
    }
    if (s.count(own)) {
        const std::vector<std::string> values = split(s.at(own), " \t,;");
        if (values.size() != nbOutputs * nbChannels)
            throw std::runtime_error(own + " in section [" + section + "] holds " + std::to_string(values.size()) + " values, the map has "
                                     + std::to_string(nbOutputs * nbChannels));
        Tensor<bool> map({nbOutputs, nbChannels}, false);
        for (std::size_t i = 0; i < values.size(); ++i)
            map.set(i % nbOutputs, i / nbOutputs, values[i] != "0");      // the file's rows are channels, its columns outputs
        return map;
    }
    bool isFunction = false;
    for (const auto& kv : s)
        isFunction = isFunction || kv.first.compare(0, 8, "Mapping.") == 0 || kv.first.compare(0, own.size() + 1, own + ".") == 0;
    Tensor<bool> map({nbOutputs, nbChannels}, !isFunction);
    if (!isFunction || map.empty())
        return map;
    auto key = [&](const std::string& both, const std::string& one) {
        for (const std::string& prefix : {own, std::string("Mapping")})
            for (const std::string& k : {both, one})
                if (s.count(prefix + "." + k))
                    return getUInt(s, prefix + "." + k, 0);
        return (unsigned int)(both == "Offset" ? 0 : 1);
    };
    std::size_t sizeX = key("Size", "SizeX"), sizeY = key("Size", "SizeY");
    const std::size_t strideX = key("Stride", "StrideX"), strideY = key("Stride", "StrideY");
    const std::size_t offsetX = key("Offset", "OffsetX"), offsetY = key("Offset", "OffsetY");
    std::size_t iterations = s.count(own + ".NbIterations") ? getUInt(s, own + ".NbIterations", 0) : getUInt(s, "Mapping.NbIterations", 0);
    if (iterations == 0) iterations = std::max(nbOutputs, nbChannels);
    if (sizeY == 0) sizeY = nbChannels;
    if (sizeX == 0) sizeX = nbOutputs;
    for (std::size_t i = 0, x = offsetX, y = offsetY; i < iterations; ++i, x += strideX, y += strideY)
        for (std::size_t px = 0; px < sizeX; ++px)
            for (std::size_t py = 0; py < sizeY; ++py)
                map.set((x + px) % nbOutputs, (y + py) % nbChannels, true);
    return map;
}
} // namespace

std::shared_ptr<DeepNet> generateFromINI(const std::string& iniText, std::string* modelOut)
{
    std::vector<std::string> order;
    std::map<std::string, Section> sections;
    std::map<std::string, std::string> inherits;
    Section global;
    std::map<std::string, std::string> variables;
    std::string current;
    std::istringstream in(iniText);
    std::string line;
    while (std::getline(in, line)) {
        const size_t c = line.find(';');
        if (c != std::string::npos) line = line.substr(0, c);
        line = trim(line);
        if (line.empty()) continue;
        if (line[0] == '[') {
            const size_t end = line.find(']');
            if (end == std::string::npos) throw std::runtime_error("Malformed section header: " + line);
            current = trim(line.substr(1, end - 1));
            const std::string parent = trim(line.substr(end + 1));
            if (!parent.empty()) inherits[current] = parent;
            if (!sections.count(current)) order.push_back(current);
            sections[current];
            continue;
        }
        const size_t eq = line.find('=');
        if (eq == std::string::npos) throw std::runtime_error("Malformed line: " + line);
        std::string key = trim(line.substr(0, eq)), value = trim(line.substr(eq + 1));
        // "$BATCH_SIZE=64" defines a variable, "${BATCH_SIZE}" takes its value (N2D2's model files size their nets this way)
        for (size_t at = value.find("${"); at != std::string::npos; at = value.find("${", at)) {
            const size_t close = value.find('}', at);
            if (close == std::string::npos) throw std::runtime_error("Malformed variable reference: " + line);
            auto var = variables.find(value.substr(at + 2, close - at - 2));
            if (var == variables.end()) throw std::runtime_error("Undefined variable in: " + line);
            value.replace(at, close - at + 1, var->second);
        }
        if (key.size() > 1 && key[0] == '$') {
            variables[key.substr(1)] = value;
            continue;
        }
        if (current.empty()) global[key] = value; else sections[current][key] = value;
    }
    std::function<Section(const std::string&, int)> resolvedAt = [&](const std::string& name, int depth) {
        Section s;
        auto ih = inherits.find(name);
        if (ih != inherits.end()) {
            // "[conv_1] conv_def other_def": the templates' keys, later ones first overridden by the section's own
            for (const std::string& baseName : split(ih->second, " \t")) {
                auto base = sections.find(baseName);
                if (base == sections.end()) throw std::runtime_error("Section [" + name + "] inherits from unknown section " + baseName);
                for (const auto& kv : base->second) s[kv.first] = kv.second;
            }
        }
        for (const auto& kv : sections[name]) s[kv.first] = kv.second;
        // "NbOutputs=[conv_pw_2]NbOutputs": the value of another section's key
        for (auto& kv : s) {
            const std::string& v = kv.second;
            const size_t close = v.find(']');
            if (v.size() > 2 && v[0] == '[' && close != std::string::npos && close + 1 < v.size()) {
                const std::string refSection = trim(v.substr(1, close - 1)), refKey = trim(v.substr(close + 1));
                if (depth > 16 || !sections.count(refSection))
                    throw std::runtime_error("Section [" + name + "]: " + kv.first + " refers to unknown section [" + refSection + "]");
                const Section other = resolvedAt(refSection, depth + 1);
                auto it = other.find(refKey);
                if (it == other.end())
                    throw std::runtime_error("Section [" + name + "]: [" + refSection + "] has no " + refKey);
                kv.second = it->second;
            }
        }
        return s;
    };
    auto resolved = [&](const std::string& name) { return resolvedAt(name, 0); };

    // src/Generator/DeepNetGenerator.cpp:124-125
    const std::string model = global.count("DefaultModel") ? global["DefaultModel"] : "Frame";
    if (modelOut) *modelOut = model;
    auto deepNet = std::make_shared<DeepNet>();
    Network net;
    std::string envName;
    for (const std::string& n : {std::string("sp"), std::string("env")})
        if (sections.count(n)) envName = n;
    if (envName.empty()) throw std::runtime_error("Missing [sp] or [env] section");
    {
        const Section env = resolved(envName);
        deepNet->setStimuli(getUInt(env, "NbChannels", 1), getUInt(env, "SizeY", 0, true, envName), getUInt(env, "SizeX", 0, true, envName),
                            getUInt(env, "BatchSize", 1));
    }
    auto makeActivation = [&](const Section& s, const std::string& name) -> std::shared_ptr<Activation> {
        auto it = s.find("ActivationFunction");
        if (it == s.end() || it->second == "None") return std::shared_ptr<Activation>();
        if (it->second == "Rectifier") {
            // src/Generator/RectifierActivationGenerator.cpp:31-43: same model key as the cells
            auto f = Registrar<RectifierActivation>::create<float>(model);
            if (!f) throw std::runtime_error("Activation model \"" + model + "\" is not valid in section [" + name + "]");
            return f();
        }
        if (it->second == "Linear") {
            auto f = Registrar<LinearActivation>::create<float>(model);
            if (!f) throw std::runtime_error("Activation model \"" + model + "\" is not valid in section [" + name + "]");
            return f();
        }
        throw std::runtime_error("Activation " + it->second + " is not on the quantized path (section [" + name + "])");
    };

    for (const std::string& name : order) {
        const Section s = resolved(name);
        if (!s.count("Type") || !s.count("Input")) continue;       // template / config sections
        const std::string type = s.at("Type");
        std::vector<std::shared_ptr<Cell> > parents;
        for (const std::string& p : split(s.at("Input"), ","))
            if (p != envName) parents.push_back(deepNet->getCell(p));
        std::shared_ptr<Cell> cell;
        if (type == "Conv") {
            auto f = Registrar<ConvCell>::create<float>(model);
            if (!f) // src/Generator/ConvCellGenerator.cpp:191-195
                throw std::runtime_error("Cell model \"" + model + "\" is not valid in section [" + name + "]");
            const std::vector<unsigned int> stride = getDims(s, "StrideDims", "Stride", "StrideX", "StrideY", 1);
            const std::vector<unsigned int> padU = getDims(s, "PaddingDims", "Padding", "PaddingX", "PaddingY", 0);
            auto conv = f(net, *deepNet, name, getDims(s, "KernelDims", "KernelSize", "KernelWidth", "KernelHeight", 1),
                          getUInt(s, "NbOutputs", 0, true, name), getDims(s, "SubSampleDims", "SubSample", "SubSampleX", "SubSampleY", 1), stride,
                          std::vector<int>{(int)padU[0], (int)padU[1]}, getDims(s, "DilationDims", "Dilation", "DilationX", "DilationY", 1),
                          makeActivation(s, name));
            if (s.count("NoBias")) conv->setParameter("NoBias", s.at("NoBias") != "0");
            cell = conv;
        } else if (type == "Fc") {
            auto f = Registrar<FcCell>::create<float>(model);
            if (!f) throw std::runtime_error("Cell model \"" + model + "\" is not valid in section [" + name + "]");
            auto fc = f(net, *deepNet, name, getUInt(s, "NbOutputs", 0, true, name), makeActivation(s, name));
            if (s.count("NoBias")) fc->setParameter("NoBias", s.at("NoBias") != "0");
            cell = fc;
        } else if (type == "Pool") {
            auto f = Registrar<PoolCell>::create<float>(model);
            if (!f) throw std::runtime_error("Cell model \"" + model + "\" is not valid in section [" + name + "]");
            const std::string pooling = s.count("Pooling") ? s.at("Pooling") : "Max";
            if (pooling != "Max" && pooling != "Average") throw std::runtime_error("Unknown pooling " + pooling + " in section [" + name + "]");
            cell = f(net, *deepNet, name, getDims(s, "PoolDims", "PoolSize", "PoolWidth", "PoolHeight", 1), getUInt(s, "NbOutputs", 0, true, name),
                     getDims(s, "StrideDims", "Stride", "StrideX", "StrideY", 1), getDims(s, "PaddingDims", "Padding", "PaddingX", "PaddingY", 0),
                     pooling == "Max" ? PoolCell::Max : PoolCell::Average, makeActivation(s, name));
        } else if (type == "ElemWise") {
            auto f = Registrar<ElemWiseCell>::create<float>(model);
            if (!f) throw std::runtime_error("Cell model \"" + model + "\" is not valid in section [" + name + "]");
            const std::string op = s.count("Operation") ? s.at("Operation") : "Sum";
            if (op != "Sum") throw std::runtime_error("ElemWise operation " + op + " is not on the quantized path (section [" + name + "])");
            // src/Generator/ElemWiseCellGenerator.cpp:50-62: Weights, Shifts (none by default), CoeffMode (PerInput by default)
            auto floats = [&](const char* key) {
                std::vector<Float_T> v;
                if (s.count(key))
                    for (const std::string& tok : split(s.at(key), " \t,"))
                        v.push_back(std::stof(tok));
                return v;
            };
            const std::string coeff = s.count("CoeffMode") ? s.at("CoeffMode") : "PerInput";
            if (coeff != "PerLayer" && coeff != "PerInput" && coeff != "PerChannel")
                throw std::runtime_error("Unknown CoeffMode " + coeff + " in section [" + name + "]");
            const ElemWiseCell::CoeffMode mode = coeff == "PerLayer" ? ElemWiseCell::PerLayer
                : (coeff == "PerInput" ? ElemWiseCell::PerInput : ElemWiseCell::PerChannel);
            cell = f(net, *deepNet, name, getUInt(s, "NbOutputs", 0, true, name), ElemWiseCell::Sum, mode, floats("Weights"), floats("Shifts"),
                     makeActivation(s, name));
        } else if (type == "Scaling") {
            auto f = Registrar<ScalingCell>::create<float>(model);
            if (!f) throw std::runtime_error("Cell model \"" + model + "\" is not valid in section [" + name + "]");
            cell = f(*deepNet, name, getUInt(s, "NbOutputs", 0, true, name), Scaling());
        } else if (type == "Softmax") {
            // The quantized graph ends at the logits: the integer cells have no Softmax (N2D2's integer exports drop it as
            // well); the section and its Target are read over.
            continue;
        } else {
            throw std::runtime_error("Cell type " + type + " is not on the quantized path (section [" + name + "])");
        }
        deepNet->addCell(cell, parents);
        // src/Generator/PoolCellGenerator.cpp:160-195, ConvCellGenerator.cpp: one map per parent, side by side
        auto mappingOverParents = [&]() {
            Tensor<bool> map({cell->getNbOutputs(), cell->getNbChannels()}, false);
            std::size_t first = 0;
            for (std::size_t k = 0; k < std::max<std::size_t>(parents.size(), 1); ++k) {
                const Cell* parent = parents.empty() ? nullptr : parents[k].get();        // no parent cell: the stimuli
                const std::size_t n = parent ? parent->getNbOutputs() : cell->getNbChannels();
                const Tensor<bool> part = generateMapping(s, name, parent ? parent->getName() : "env", cell->getNbOutputs(), n);
                for (std::size_t o = 0; o < cell->getNbOutputs(); ++o)
                    for (std::size_t ch = 0; ch < n; ++ch)
                        map.set(o, first + ch, part.at(o, ch));
                first += n;
            }
            return map;
        };
        if (type == "Pool") {
            auto pool = std::dynamic_pointer_cast<PoolCell_Frame_HIP<float> >(cell);
            if (pool) pool->setMapping(mappingOverParents());
        }
        if (type == "Conv") {
            const unsigned int perGroup = getUInt(s, "Mapping.ChannelsPerGroup", 0);
            const unsigned int groups = perGroup ? cell->getNbChannels() / perGroup : getUInt(s, "Mapping.NbGroups", 1);
            // the reference builds the groups per parent and refuses channels they do not divide
            // (src/Generator/MappingGenerator.cpp:110-128)
            if ((perGroup || s.count("Mapping.NbGroups")) && (groups == 0 || cell->getNbChannels() % groups != 0))
                throw std::runtime_error("Mapping.NbGroups must be a multiple of the number of input channels in section [" + name + "]");
            if (groups > 1 && parents.size() > 1)
                throw std::runtime_error("Mapping: a grouped Conv with several parents is not supported in section [" + name
                                         + "] (the reference lays one group structure per parent side by side)");
            if (groups > 1)
                std::dynamic_pointer_cast<ConvCell>(cell)->setNbGroups(groups);
            else if (!perGroup && !s.count("Mapping.NbGroups")) {
                const Tensor<bool> map = mappingOverParents();      // a map written out or stepped along the diagonal
                bool full = true;
                for (std::size_t o = 0; full && o < map.dimX(); ++o)
                    for (std::size_t ch = 0; full && ch < map.dimY(); ++ch)
                        full = map.at(o, ch);
                if (!full) std::dynamic_pointer_cast<ConvCell>(cell)->setMapping(map);
            }
        }
    }
    return deepNet;
}

// Every output of block g = o / (O / G) must see exactly the channels [g L, (g + 1) L), L being the number of leading
// channels the first output sees.
std::size_t Cell::getNbGroups(const Tensor<bool>& map, bool* isRegular)
{
    const std::size_t nbOutputs = map.dimX(), nbChannels = map.dimY();
    if (isRegular) *isRegular = true;
    std::size_t width = 0;
    while (width < nbChannels && map.at(0, width))
        ++width;
    if (width == 0)
        return 0;
    const std::size_t groups = nbChannels / width;
    bool regular = nbChannels % width == 0 && nbOutputs % groups == 0;
    const std::size_t perGroup = regular ? nbOutputs / groups : 1;
    for (std::size_t o = 0; regular && o < nbOutputs; ++o)
        for (std::size_t ch = 0; regular && ch < nbChannels; ++ch)
            regular = map.at(o, ch) == (ch / width == o / perGroup);
    if (regular)
        return groups;
    if (isRegular) *isRegular = false;
    return getNbGroupsHandMade(map);
}

// Outputs that share a channel, directly or through other outputs, are one group: channels are merged into sets as the
// outputs connect them, and every output names the set of its channels.
std::size_t Cell::getNbGroupsHandMade(const Tensor<bool>& map)
{
    const std::size_t nbOutputs = map.dimX(), nbChannels = map.dimY();
    std::vector<std::size_t> parent(nbChannels);
    for (std::size_t ch = 0; ch < nbChannels; ++ch) parent[ch] = ch;
    auto root = [&](std::size_t ch) {
        while (parent[ch] != ch) { parent[ch] = parent[parent[ch]]; ch = parent[ch]; }
        return ch;
    };
    const std::size_t none = nbChannels;
    std::vector<std::size_t> firstChannel(nbOutputs, none);
    bool connectedSeen = false;
    for (std::size_t o = 0; o < nbOutputs; ++o) {
        for (std::size_t ch = 0; ch < nbChannels; ++ch) {
            if (!map.at(o, ch)) continue;
            if (firstChannel[o] == none) firstChannel[o] = ch;
            else parent[root(ch)] = root(firstChannel[o]);
        }
        if (firstChannel[o] != none)
            connectedSeen = true;
        else if (connectedSeen)
            throw std::runtime_error("Cell::getNbGroupsHandMade(): an output without any connection behind a connected one "
                                     "(the reference does not return on such a map)");
    }
    std::vector<bool> counted(nbChannels, false);
    std::size_t groups = 0;
    for (std::size_t o = 0; o < nbOutputs; ++o) {
        if (firstChannel[o] == none) continue;
        const std::size_t r = root(firstChannel[o]);
        if (!counted[r]) { counted[r] = true; ++groups; }
    }
    return groups;
}

void ConvCell::setMapping(const Tensor<bool>& map)
{
    if (map.dimX() != mNbOutputs || (mNbChannels != 0 && map.dimY() != mNbChannels))
        throw std::runtime_error("ConvCell::setMapping(): the map of " + mName + " must be {nbOutputs, nbChannels}");
    bool regular = true;
    const std::size_t groups = getNbGroups(map, &regular);
    if (groups == 0)
        throw std::runtime_error("ConvCell::setMapping(): the first output of " + mName + " is not connected");
    if (!regular && groups > 1 && map.dimY() % groups != 0)
        throw std::runtime_error("ConvCell::setMapping(): the " + std::to_string(groups) + " groups of the map of " + mName
                                 + " do not divide its channels");
    setNbGroups((unsigned int)groups);
    if (!regular)
        mIrregularMap = map;
}

Tensor<Float_T> ConvCell::fullConnectionWeights() const
{
    const std::size_t kw = mKernelDims[0], kh = mKernelDims[1], taps = kw * kh, slices = weightSlices();
    Tensor<Float_T> full({kw, kh, (std::size_t)mNbChannels, (std::size_t)mNbOutputs}, Float_T(0));
    for (std::size_t o = 0; o < mNbOutputs; ++o) {
        const std::vector<std::size_t> from = connectedSlices(o);
        std::size_t n = 0;
        for (std::size_t ch = 0; ch < mNbChannels; ++ch) {
            if (!mIrregularMap.at(o, ch)) continue;
            for (std::size_t t = 0; t < taps; ++t)
                full(t + taps * (ch + mNbChannels * o)) = mWeights(t + taps * (from[n] + slices * o));
            ++n;
        }
    }
    return full;
}

} // namespace N2D2
