// Float cells of the Frame_HIP model for quantization-aware training (see frame_hip_train.hpp).
#include <hip/hip_runtime_api.h>

#include "frame_hip_train.hpp"

namespace N2D2 {

static void checkHipT(hipError_t e, const char* what)
{
    if (e != hipSuccess)
        throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

// --------------------------------------------------------------- DeviceFloats
DeviceFloats::~DeviceFloats()
{
    if (mData) (void)hipFree(mData);
}

void DeviceFloats::resize(const std::vector<size_t>& dims)
{
    std::vector<size_t> d = dims;
    while (d.size() < 4) d.push_back(1);
    if (mData) (void)hipFree(mData);
    mData = nullptr;
    mDims = d;
    mValid = false;
    if (size() == 0)
        return;
    checkHipT(hipMalloc((void**)&mData, size() * sizeof(float)), "DeviceFloats::resize()");
    checkHipT(hipMemset(mData, 0, size() * sizeof(float)), "DeviceFloats::resize()");
}

void DeviceFloats::fromHost(const float* host, size_t n)
{
    if (n != size())
        throw std::runtime_error("DeviceFloats::fromHost(): size mismatch");
    checkHipT(hipMemcpy(mData, host, n * sizeof(float), hipMemcpyHostToDevice), "DeviceFloats::fromHost()");
}

void DeviceFloats::fromHost(const Tensor<Float_T>& host)
{
    if (host.dims() != mDims)
        resize(host.dims());
    fromHost(host.data(), host.size());
}

Tensor<Float_T> DeviceFloats::toHost() const
{
    Tensor<Float_T> host(mDims);
    if (size() > 0)
        checkHipT(hipMemcpy(host.data(), mData, size() * sizeof(float), hipMemcpyDeviceToHost), "DeviceFloats::toHost()");
    return host;
}

// -------------------------------------------------------- Cell_FrameTrain_HIP
Cell_FrameTrain_HIP::~Cell_FrameTrain_HIP()
{
    if (mLoss) (void)hipFree(mLoss);
    if (mLossWorkspace) (void)hipFree(mLossWorkspace);
}

void Cell_FrameTrain_HIP::addInput(Cell_FrameTrain_HIP* parent)
{
    if (!parent)
        throw std::runtime_error("Cell " + mName + ": null parent");
    if (mIn)
        throw std::runtime_error("Cell " + mName + ": the float Frame_HIP cells take one input tensor");
    if (parent->mOutputs.empty())
        throw std::runtime_error("Cell " + mName + ": initialize() the parent cell " + parent->getName() + " first");
    mParents.push_back(parent);
    mIn = &parent->mOutputs;
    mDiffOut = &parent->mDiffInputs;
    mNbChannels = parent->getNbOutputs();
    mInW = parent->getOutputsWidth();
    mInH = parent->getOutputsHeight();
    setOutputsDims();
}

void Cell_FrameTrain_HIP::addInput(DeviceFloats& inputs, DeviceFloats& diffOutputs)
{
    if (mIn)
        throw std::runtime_error("Cell " + mName + ": the float Frame_HIP cells take one input tensor");
    if (inputs.empty())
        throw std::runtime_error("Cell " + mName + ": empty input tensor");
    if (!diffOutputs.empty() && diffOutputs.dims() != inputs.dims())
        throw std::runtime_error("Cell " + mName + ": inputs and diffOutputs of different sizes");
    mParents.push_back(nullptr);
    mIn = &inputs;
    mDiffOut = &diffOutputs;
    mNbChannels = (unsigned int)inputs.dimZ();
    mInW = (unsigned int)inputs.dimX();
    mInH = (unsigned int)inputs.dimY();
    setOutputsDims();
}

void Cell_FrameTrain_HIP::allocateOutputs()
{
    if (!mIn)
        throw std::runtime_error("Cell " + mName + ": no input");
    const std::vector<size_t> dims = {mOutW, mOutH, mNbOutputs, mIn->dimB()};
    mOutputs.resize(dims);
    mDiffInputs.resize(dims);
}

void Cell_FrameTrain_HIP::activationPropagate(bool inference)
{
    if (!mActivation)
        return;
    // RectifierActivation_Frame<T>::propagate / LinearActivation_Frame<T>::propagate of an unquantized cell
    // (include/Activation/RectifierActivation_Frame.hpp:55-87, LinearActivation_Frame.hpp:56-81), Scaling NONE
    if (mActivation->getActivationScaling().getMode() != ScalingMode::NONE)
        throw std::runtime_error("Cell " + mName + ": an activation Scaling belongs to the integer cells (model Frame_HIP)");
    if (mActivation->abiKind() == N2D2HIP_ACT_RECTIFIER)
        checkStatus(n2d2hip_rectifier_f32_forward(mOutputs.data(), mOutputs.size(), mActivation->leakSlope(), (float)mActivation->clipping(), mStream));
    else if (mActivation->clipping() != 0.0)
        throw std::runtime_error("Cell " + mName + ": LinearActivation Clipping is not supported by the float Frame_HIP cells");
    if (mActivation->getQuantizer())
        mActivation->getQuantizer()->propagate(mOutputs.data(), mOutputs.size(), inference);
}

void Cell_FrameTrain_HIP::activationBackPropagate()
{
    if (!mActivation)
        return;
    // in place on mDiffInputs: the quantizer first, then the activation's own derivative taken on the cell's outputs
    // as they are after the quantizer (RectifierActivation_Frame.hpp:89-130, LinearActivation_Frame.hpp:83-123)
    if (mActivation->getQuantizer())
        mActivation->getQuantizer()->back_propagate(mDiffInputs.data(), mDiffInputs.data(), mDiffInputs.size());
    if (mActivation->abiKind() == N2D2HIP_ACT_RECTIFIER)
        checkStatus(n2d2hip_rectifier_f32_backward(mOutputs.data(), mDiffInputs.data(), mDiffInputs.data(), mDiffInputs.size(),
                                                   mActivation->leakSlope(), (float)mActivation->clipping(), mStream));
}

void Cell_FrameTrain_HIP::activationUpdate()
{
    if (mActivation && mActivation->getQuantizer())
        mActivation->getQuantizer()->update((unsigned int)mIn->dimB());
}

double Cell_FrameTrain_HIP::applyLoss()
{
    const size_t n = mOutputs.size();
    if (!mLoss)
        checkHipT(hipMalloc((void**)&mLoss, sizeof(double)), "Cell_FrameTrain_HIP::applyLoss()");
    const size_t need = n2d2hip_loss_workspace_bytes(n);
    if (mLossWorkspaceBytes < need) {
        if (mLossWorkspace) (void)hipFree(mLossWorkspace);
        mLossWorkspace = nullptr;
        checkHipT(hipMalloc(&mLossWorkspace, need), "Cell_FrameTrain_HIP::applyLoss()");
        mLossWorkspaceBytes = need;
    }
    // target and diff are the same buffer: each element is read, then written, by one thread
    checkStatus(n2d2hip_loss_f32(mDiffInputs.data(), mOutputs.data(), mDiffInputs.data(), n, (int)mOutputs.dimB(), mLoss,
                                 mLossWorkspace, mLossWorkspaceBytes, mStream));
    mDiffInputs.setValid();
    double loss = 0.0;
    checkHipT(hipMemcpy(&loss, mLoss, sizeof(double), hipMemcpyDeviceToHost), "Cell_FrameTrain_HIP::applyLoss()");
    return loss;
}

// ------------------------------------------------ WeightedCell_FrameTrain_HIP
WeightedCell_FrameTrain_HIP::WeightedCell_FrameTrain_HIP()
    : mWeightsSolver(std::make_shared<SGDSolver_Frame_HIP<float> >()), mBiasSolver(std::make_shared<SGDSolver_Frame_HIP<float> >())
{
}

void WeightedCell_FrameTrain_HIP::initializeWeights(const Tensor<Float_T>& weights, Tensor<Float_T>& biases, bool noBias, size_t quantizerOutputsSize)
{
    allocateOutputs();
    mDevW.fromHost(weights);
    mDevDiffW.resize(weights.dims());
    if (!noBias) {
        if (biases.size() != mNbOutputs)
            biases.resize({mNbOutputs}, 0.0f);
        mDevBias.resize({mNbOutputs});
        mDevBias.fromHost(biases.data(), mNbOutputs);
        mDevDiffBias.resize({mNbOutputs});
    }
    if (mQuantizer) {
        // ConvCell_Frame / FcCell_Frame::initialize hand each weight tensor and its gradient to the quantizer
        // (src/Cell/ConvCell_Frame.cpp:288-300, src/Cell/FcCell_Frame.cpp:106-112); outputsSize = dimB * dimY * dimX of
        // the weight tensor as the reference shapes it
        mQuantizer->addWeights(mDevW.data(), mDevDiffW.data(), mDevW.size(), quantizerOutputsSize);
        mQuantizer->initialize();
    }
}

void WeightedCell_FrameTrain_HIP::propagateWeighted(bool inference, bool noBias)
{
    if (mQuantizer)
        mQuantizer->propagate();
    const n2d2hip_conv_desc d = desc();
    const float* w = mQuantizer ? mQuantizer->getQuantizedWeights(0) : mDevW.data();
    const size_t need = n2d2hip_conv2d_f32_workspace_bytes(&d, (int)mIn->dimB(), (int)mInH, (int)mInW);
    if (need > mWorkspace.size() * sizeof(float))
        mWorkspace.resize({(need + sizeof(float) - 1) / sizeof(float)});
    // a quantizer passes the biases through (quantize_bias_propagate copies them)
    checkStatus(n2d2hip_conv2d_f32_forward(&d, (int)mIn->dimB(), (int)mInH, (int)mInW, mIn->data(), w, noBias ? nullptr : mDevBias.data(), 0.0f,
                                           mOutputs.data(), mWorkspace.data(), mWorkspace.size() * sizeof(float), mStream));
    activationPropagate(inference);
    mDiffInputs.clearValid();
    mDevDiffW.clearValid();
    mDevDiffBias.clearValid();
}

void WeightedCell_FrameTrain_HIP::backPropagateWeighted(bool noBias)
{
    if (!mDiffInputs.isValid())
        return;
    activationBackPropagate();
    const n2d2hip_conv_desc d = desc();
    const int B = (int)mIn->dimB();
    {
        const float beta = mWeightsSolver->isNewIteration() ? 0.0f : 1.0f;
        checkStatus(n2d2hip_conv2d_f32_backward_filter(&d, B, (int)mInH, (int)mInW, mIn->data(), mDiffInputs.data(), beta, mDevDiffW.data(),
                                                       mWorkspace.data(), mWorkspace.size() * sizeof(float), mStream));
        mDevDiffW.setValid();
    }
    if (!noBias) {
        const float beta = mBiasSolver->isNewIteration() ? 0.0f : 1.0f;
        checkStatus(n2d2hip_conv2d_f32_backward_bias(B, (int)mNbOutputs, (int)mOutH, (int)mOutW, mDiffInputs.data(), beta, mDevDiffBias.data(), mStream));
        mDevDiffBias.setValid();
    }
    if (mDiffOut && !mDiffOut->empty()) {
        const float beta = mDiffOut->isValid() ? 1.0f : 0.0f;
        const float* w = mQuantizer ? mQuantizer->getQuantizedWeights(0) : mDevW.data();
        checkStatus(n2d2hip_conv2d_f32_backward_data(&d, B, (int)mInH, (int)mInW, w, mDiffInputs.data(), beta, mDiffOut->data(),
                                                     mWorkspace.data(), mWorkspace.size() * sizeof(float), mStream));
        mDiffOut->setValid();
    }
    if (mQuantizer)
        mQuantizer->back_propagate();
}

void WeightedCell_FrameTrain_HIP::updateWeighted(bool noBias)
{
    const unsigned int batch = (unsigned int)mIn->dimB();
    if (mDevDiffW.isValid())
        mWeightsSolver->update(mDevW.data(), mQuantizer ? mQuantizer->getDiffFullPrecisionWeights(0) : mDevDiffW.data(), mDevW.size(), batch, mStream);
    if (!noBias && mDevDiffBias.isValid())
        mBiasSolver->update(mDevBias.data(), mDevDiffBias.data(), mDevBias.size(), batch, mStream);
    if (mQuantizer)
        mQuantizer->update(batch);
    activationUpdate();
}

Tensor<Float_T> WeightedCell_FrameTrain_HIP::getQuantizedWeights() const
{
    Tensor<Float_T> host(mDevW.dims());
    const float* src = mQuantizer ? mQuantizer->getQuantizedWeights(0) : mDevW.data();
    checkHipT(hipMemcpy(host.data(), src, host.size() * sizeof(float), hipMemcpyDeviceToHost), "WeightedCell_FrameTrain_HIP::getQuantizedWeights()");
    return host;
}

QATCellParameters WeightedCell_FrameTrain_HIP::getQATCellParameters()
{
    QATCellParameters p;
    p.quantWeights = getQuantizedWeights();
    synchronizeWeightsToHost();
    if (!mDevBias.empty())
        p.biases = mDevBias.toHost();
    if (mQuantizer) {
        p.weightsRange = mQuantizer->getRange();
        p.defaultQuantMode = mQuantizer->getQuantMode() == QuantizerCell::Default;
        if (auto sat = std::dynamic_pointer_cast<SATQuantizerCell_Frame_HIP<float> >(mQuantizer))
            p.satScaling = sat->getScaling() ? (double)sat->getStats(0).second : 1.0;
    }
    return p;
}

// ------------------------------------------------------ ConvCell_FrameTrain_HIP
template <class T>
ConvCell_FrameTrain_HIP<T>::ConvCell_FrameTrain_HIP(const DeepNet& /*deepNet*/, const std::string& name, const std::vector<unsigned int>& kernelDims,
                                                    unsigned int nbOutputs, const std::vector<unsigned int>& subSampleDims,
                                                    const std::vector<unsigned int>& strideDims, const std::vector<int>& paddingDims,
                                                    const std::vector<unsigned int>& dilationDims, const std::shared_ptr<Activation>& activation)
    : Cell(name, nbOutputs), ConvCell(kernelDims, subSampleDims, strideDims, paddingDims, dilationDims)
{
    if (mSubSampleDims[0] != 1 || mSubSampleDims[1] != 1)
        throw std::runtime_error("ConvCell: sub-sampling is not supported by the learning cells of Frame_HIP_QAT");
    mActivation = activation;
}

template <class T>
ConvCell_FrameTrain_HIP<T>::~ConvCell_FrameTrain_HIP() {}

template <class T>
void ConvCell_FrameTrain_HIP<T>::setOutputsDims()
{
    // src/Cell/ConvCell.cpp:1169-1195
    const unsigned int in[2] = {mInW, mInH};
    unsigned int out[2];
    for (int dim = 0; dim < 2; ++dim) {
        const int kernelExtent = (int)(mDilationDims[dim] * (mKernelDims[dim] - 1) + 1);
        out[dim] = (unsigned int)std::floor(((int)in[dim] + 2 * mPaddingDims[dim] - kernelExtent + (int)mStrideDims[dim]) / (double)mStrideDims[dim]);
    }
    mOutW = out[0];
    mOutH = out[1];
}

template <class T>
n2d2hip_conv_desc ConvCell_FrameTrain_HIP<T>::desc() const
{
    n2d2hip_conv_desc d = {};
    d.C = (int)mNbChannels;
    d.O = (int)mNbOutputs;
    d.kW = (int)mKernelDims[0];
    d.kH = (int)mKernelDims[1];
    d.strideX = (int)mStrideDims[0];
    d.strideY = (int)mStrideDims[1];
    d.padL = d.padR = mPaddingDims[0];
    d.padT = d.padB = mPaddingDims[1];
    d.dilX = (int)mDilationDims[0];
    d.dilY = (int)mDilationDims[1];
    d.groups = (int)mNbGroups;
    return d;
}

template <class T>
void ConvCell_FrameTrain_HIP<T>::initialize()
{
    const std::vector<size_t> wdims = {mKernelDims[0], mKernelDims[1], mNbChannels / mNbGroups, mNbOutputs};
    if (mWeights.dims() != wdims)
        throw std::runtime_error("ConvCell_FrameTrain_HIP " + mName + ": setWeights() with a {kW, kH, C/groups, O} tensor before initialize()");
    initializeWeights(mWeights, mBias, mNoBias, (size_t)mNbOutputs * mKernelDims[1] * mKernelDims[0]);
}

template <class T>
void ConvCell_FrameTrain_HIP<T>::synchronizeWeightsToHost()
{
    mWeights = mDevW.toHost();
    if (!mNoBias) {
        const Tensor<Float_T> b = mDevBias.toHost();
        mBias.resize({mNbOutputs});
        for (size_t i = 0; i < mNbOutputs; ++i) mBias(i) = b(i);
    }
}

template class ConvCell_FrameTrain_HIP<float>;
template <> Registrar<ConvCell> ConvCell_FrameTrain_HIP<float>::mRegistrar("Frame_HIP_QAT", ConvCell_FrameTrain_HIP<float>::create,
                                                                           Registrar<ConvCell>::Type<float>());

// -------------------------------------------------------- FcCell_FrameTrain_HIP
template <class T>
FcCell_FrameTrain_HIP<T>::FcCell_FrameTrain_HIP(const DeepNet& /*deepNet*/, const std::string& name, unsigned int nbOutputs,
                                                const std::shared_ptr<Activation>& activation)
    : Cell(name, nbOutputs)
{
    mActivation = activation;
}

template <class T>
n2d2hip_conv_desc FcCell_FrameTrain_HIP<T>::desc() const
{
    // the convolution whose kernel spans the input: weights [O][C*H*W] in CHW order are an OCHW kernel
    n2d2hip_conv_desc d = {};
    d.C = (int)mNbChannels;
    d.O = (int)mNbOutputs;
    d.kW = (int)mInW;
    d.kH = (int)mInH;
    d.strideX = d.strideY = 1;
    d.dilX = d.dilY = 1;
    d.groups = 1;
    return d;
}

template <class T>
void FcCell_FrameTrain_HIP<T>::initialize()
{
    const size_t K = (size_t)mNbChannels * mInH * mInW;
    if (mWeights.size() != K * mNbOutputs)
        throw std::runtime_error("FcCell_FrameTrain_HIP " + mName + ": setWeights() with a {K, O} tensor, K = C*H*W, before initialize()");
    // the reference shapes an FcCell's synapses {1, 1, K, O} (src/Cell/FcCell_Frame.cpp:99-102): dimB * dimY * dimX = O
    initializeWeights(mWeights, mBias, mNoBias, mNbOutputs);
}

template <class T>
void FcCell_FrameTrain_HIP<T>::synchronizeWeightsToHost()
{
    const Tensor<Float_T> w = mDevW.toHost();
    for (size_t i = 0; i < w.size(); ++i) mWeights(i) = w(i);
    if (!mNoBias) {
        const Tensor<Float_T> b = mDevBias.toHost();
        mBias.resize({mNbOutputs});
        for (size_t i = 0; i < mNbOutputs; ++i) mBias(i) = b(i);
    }
}

template class FcCell_FrameTrain_HIP<float>;
template <> Registrar<FcCell> FcCell_FrameTrain_HIP<float>::mRegistrar("Frame_HIP_QAT", FcCell_FrameTrain_HIP<float>::create,
                                                                       Registrar<FcCell>::Type<float>());

// ------------------------------------------------ ActivationCell_FrameTrain_HIP
const char* ActivationCell::Type = "Activation";

template <class T>
ActivationCell_FrameTrain_HIP<T>::ActivationCell_FrameTrain_HIP(const DeepNet& /*deepNet*/, const std::string& name, unsigned int nbOutputs,
                                                                const std::shared_ptr<Activation>& activation)
    : Cell(name, nbOutputs)
{
    mActivation = activation;
}

template <class T>
void ActivationCell_FrameTrain_HIP<T>::initialize()
{
    if (!mActivation)
        throw std::runtime_error("ActivationCell_FrameTrain_HIP " + mName + ": no activation");
    if (mNbChannels != mNbOutputs)
        throw std::runtime_error("ActivationCell_FrameTrain_HIP " + mName + ": the number of outputs must be the number of input channels");
    allocateOutputs();
}

template <class T>
void ActivationCell_FrameTrain_HIP<T>::propagate(bool inference)
{
    checkHipT(hipMemcpyAsync(mOutputs.data(), mIn->data(), mOutputs.size() * sizeof(float), hipMemcpyDeviceToDevice, (hipStream_t)mStream),
              "ActivationCell_FrameTrain_HIP::propagate()");
    activationPropagate(inference);
    mDiffInputs.clearValid();
}

template <class T>
void ActivationCell_FrameTrain_HIP<T>::backPropagate()
{
    if (!mDiffInputs.isValid())
        return;
    if (!mDiffOut || mDiffOut->empty())
        return;
    // out of place in the reference (mDiffInputs -> diffOutput); the quantizers' gradients come out the same
    activationBackPropagate();
    checkHipT(hipMemcpyAsync(mDiffOut->data(), mDiffInputs.data(), mDiffInputs.size() * sizeof(float), hipMemcpyDeviceToDevice, (hipStream_t)mStream),
              "ActivationCell_FrameTrain_HIP::backPropagate()");
    mDiffOut->setValid();
}

template class ActivationCell_FrameTrain_HIP<float>;
template <> Registrar<ActivationCell> ActivationCell_FrameTrain_HIP<float>::mRegistrar("Frame_HIP_QAT", ActivationCell_FrameTrain_HIP<float>::create,
                                                                                       Registrar<ActivationCell>::Type<float>());

// ------------------------------------------------- BatchNormCell_FrameTrain_HIP
const char* BatchNormCell::Type = "BatchNorm";

void BatchNormCell::setParameter(const std::string& name, double value)
{
    if (name == "Epsilon") {
        if (!(value > 0.0))
            throw std::runtime_error("BatchNormCell " + mName + ": Epsilon must be positive");
        mEpsilon = value;
    } else if (name == "MovingAverageMomentum")
        mMovingAverageMomentum = value;
    else
        throw std::runtime_error("Parameter does not exist: " + name);
}

template <class T>
BatchNormCell_FrameTrain_HIP<T>::BatchNormCell_FrameTrain_HIP(const DeepNet& /*deepNet*/, const std::string& name, unsigned int nbOutputs,
                                                              const std::shared_ptr<Activation>& activation)
    : Cell(name, nbOutputs), mScaleSolver(std::make_shared<SGDSolver_Frame_HIP<float> >()),
      mBiasSolver(std::make_shared<SGDSolver_Frame_HIP<float> >()), mLearned(false)
{
    mActivation = activation;
}

template <class T>
void BatchNormCell_FrameTrain_HIP<T>::set(DeviceFloats& dev, std::vector<Float_T>& host, const std::vector<Float_T>& v)
{
    if (v.size() != mNbOutputs)
        throw std::runtime_error("BatchNormCell_FrameTrain_HIP " + mName + ": one value per output expected");
    host = v;
    if (!dev.empty())
        dev.fromHost(v.data(), v.size());
}

template <class T>
std::vector<Float_T> BatchNormCell_FrameTrain_HIP<T>::get(const DeviceFloats& dev, const std::vector<Float_T>& host) const
{
    if (dev.empty())
        return host;
    checkHipT(hipStreamSynchronize((hipStream_t)mStream), "BatchNormCell_FrameTrain_HIP: synchronize");
    const Tensor<Float_T> t = dev.toHost();
    return std::vector<Float_T>(t.data(), t.data() + t.size());
}

template <class T>
BatchNormParameters BatchNormCell_FrameTrain_HIP<T>::getBatchNormParameters() const
{
    BatchNormParameters p;
    const std::vector<Float_T> s = getScales(), b = getBiases(), m = getMeans(), v = getVariances();
    p.scales.assign(s.begin(), s.end());
    p.biases.assign(b.begin(), b.end());
    p.means.assign(m.begin(), m.end());
    p.variances.assign(v.begin(), v.end());
    p.epsilon = mEpsilon;
    if (mActivation && mActivation->getQuantizer()) {
        if (auto sat = std::dynamic_pointer_cast<SATQuantizerActivation_Frame_HIP<float> >(mActivation->getQuantizer())) {
            p.actRange = sat->getRange();
            p.actAlpha = sat->getAlpha();
        }
    }
    return p;
}

template <class T>
void BatchNormCell_FrameTrain_HIP<T>::initialize()
{
    if (mNbChannels != mNbOutputs)
        throw std::runtime_error("BatchNormCell_FrameTrain_HIP " + mName + ": the number of outputs must be the number of input channels");
    allocateOutputs();
    const std::vector<size_t> dims = {1, 1, (size_t)mNbOutputs, 1};
    struct Init { DeviceFloats* dev; std::vector<Float_T>* host; Float_T value; };
    const Init params[] = {{&mScale, &mHostScale, 1.0f}, {&mBias, &mHostBias, 0.0f}, {&mMean, &mHostMean, 0.0f}, {&mVariance, &mHostVariance, 0.0f}};
    for (const Init& p : params) {
        p.dev->resize(dims);
        if (p.host->empty())
            p.host->assign(mNbOutputs, p.value);
        p.dev->fromHost(p.host->data(), p.host->size());
    }
    for (DeviceFloats* d : {&mSavedMean, &mSavedVariance, &mDiffScale, &mDiffBias, &mDiffSavedMean, &mDiffSavedVariance})
        d->resize(dims);
    const size_t bytes = n2d2hip_batchnorm_f32_workspace_bytes((int)mIn->dimB(), (int)mNbOutputs, (int)mInH, (int)mInW);
    mWorkspace.resize({(bytes + sizeof(float) - 1) / sizeof(float), 1, 1, 1});
}

template <class T>
void BatchNormCell_FrameTrain_HIP<T>::propagate(bool inference)
{
    checkStatus(n2d2hip_batchnorm_f32_forward((int)mIn->dimB(), (int)mNbOutputs, (int)mInH, (int)mInW, mIn->data(), mScale.data(), mBias.data(),
                                              mMean.data(), mVariance.data(), mSavedMean.data(), mSavedVariance.data(), mEpsilon, mMovingAverageMomentum,
                                              inference ? 1 : 0, mOutputs.data(), mWorkspace.data(), mWorkspace.size() * sizeof(float), mStream));
    if (!inference && mMovingAverageMomentum != 0.0)
        mLearned = true;
    activationPropagate(inference);
    mDiffInputs.clearValid();
    mDiffScale.clearValid();
    mDiffBias.clearValid();
}

template <class T>
void BatchNormCell_FrameTrain_HIP<T>::backPropagate()
{
    if (!mDiffInputs.isValid())
        return;
    if (!mLearned)
        throw std::runtime_error("BatchNormCell_FrameTrain_HIP " + mName + ": backPropagate() needs the batch statistics of a learning propagate()");
    activationBackPropagate();
    const float betaScale = mScaleSolver->isNewIteration() ? 0.0f : 1.0f;
    const float betaBias = mBiasSolver->isNewIteration() ? 0.0f : 1.0f;
    const bool toInput = mDiffOut && !mDiffOut->empty();
    // A gradient another consumer of the same input has already written is added to, as the reference does with its
    // `isValid * diffOutputs` term (src/Cell/BatchNormCell_Frame.cpp:458-488): this cell's part goes to a buffer of its own
    // first and is then added in one pass.
    const bool accumulate = toInput && mDiffOut->isValid();
    if (accumulate && mDiffOwn.size() != mDiffOut->size())
        mDiffOwn.resize(mDiffOut->dims());
    float* dst = !toInput ? nullptr : accumulate ? mDiffOwn.data() : mDiffOut->data();
    checkStatus(n2d2hip_batchnorm_f32_backward((int)mIn->dimB(), (int)mNbOutputs, (int)mInH, (int)mInW, mIn->data(), mScale.data(), mSavedMean.data(),
                                               mSavedVariance.data(), mEpsilon, mDiffInputs.data(), betaScale, mDiffScale.data(), betaBias,
                                               mDiffBias.data(), mDiffSavedMean.data(), mDiffSavedVariance.data(), dst,
                                               mWorkspace.data(), mWorkspace.size() * sizeof(float), mStream));
    if (accumulate)
        checkStatus(n2d2hip_elemwise_sum_f32_backward(mDiffOut->size(), 1.0f, mDiffOwn.data(), 1.0f, mDiffOut->data(), mStream));
    if (toInput)
        mDiffOut->setValid();
    mDiffScale.setValid();
    mDiffBias.setValid();
}

template <class T>
void BatchNormCell_FrameTrain_HIP<T>::update()
{
    const unsigned int batch = (unsigned int)mIn->dimB();
    if (mDiffScale.isValid())
        mScaleSolver->update(mScale.data(), mDiffScale.data(), mScale.size(), batch, mStream);
    if (mDiffBias.isValid())
        mBiasSolver->update(mBias.data(), mDiffBias.data(), mBias.size(), batch, mStream);
    activationUpdate();
}

template class BatchNormCell_FrameTrain_HIP<float>;
template <> Registrar<BatchNormCell> BatchNormCell_FrameTrain_HIP<float>::mRegistrar("Frame_HIP_QAT", BatchNormCell_FrameTrain_HIP<float>::create,
                                                                                     Registrar<BatchNormCell>::Type<float>());

// ------------------------------------------------------ PoolCell_FrameTrain_HIP
template <class T>
PoolCell_FrameTrain_HIP<T>::PoolCell_FrameTrain_HIP(const DeepNet& /*deepNet*/, const std::string& name, const std::vector<unsigned int>& poolDims,
                                                    unsigned int nbOutputs, const std::vector<unsigned int>& strideDims,
                                                    const std::vector<unsigned int>& paddingDims, Pooling pooling,
                                                    const std::shared_ptr<Activation>& activation)
    : Cell(name, nbOutputs), PoolCell(poolDims, strideDims, paddingDims, pooling), mArgMax(nullptr)
{
    if (poolDims.size() != 2 || strideDims.size() != 2 || paddingDims.size() != 2)
        throw std::runtime_error("PoolCell_FrameTrain_HIP " + name + ": two-dimensional pooling expected");
    mActivation = activation;
}

template <class T>
PoolCell_FrameTrain_HIP<T>::~PoolCell_FrameTrain_HIP()
{
    if (mArgMax)
        (void)hipFree(mArgMax);
}

template <class T>
void PoolCell_FrameTrain_HIP<T>::setOutputsDims()
{
    // PoolCell::setOutputsDims (src/Cell/PoolCell.cpp:219-240)
    mOutW = (unsigned int)(((int)mInW + 2 * (int)mPaddingDims[0] - (int)mPoolDims[0] + (int)mStrideDims[0]) / (double)mStrideDims[0]);
    mOutH = (unsigned int)(((int)mInH + 2 * (int)mPaddingDims[1] - (int)mPoolDims[1] + (int)mStrideDims[1]) / (double)mStrideDims[1]);
}

template <class T>
void PoolCell_FrameTrain_HIP<T>::initialize()
{
    if (mNbChannels != mNbOutputs)
        throw std::runtime_error("PoolCell_FrameTrain_HIP " + mName + ": one output per input channel expected (the unit mapping)");
    allocateOutputs();
    if (mArgMax) {
        (void)hipFree(mArgMax);
        mArgMax = nullptr;
    }
    if (mPooling == Max)
        checkHipT(hipMalloc((void**)&mArgMax, mOutputs.size() * sizeof(int)), "PoolCell_FrameTrain_HIP::initialize()");
}

template <class T>
void PoolCell_FrameTrain_HIP<T>::propagate(bool inference)
{
    if (mPooling == Max)
        checkStatus(n2d2hip_pool_max_f32_forward((int)mIn->dimB(), (int)mNbOutputs, (int)mInH, (int)mInW, (int)mPoolDims[0], (int)mPoolDims[1],
                                                 (int)mStrideDims[0], (int)mStrideDims[1], (int)mPaddingDims[0], (int)mPaddingDims[1], mIn->data(),
                                                 mOutputs.data(), mArgMax, mStream));
    else        // Average counts the padding, as PoolCell_Frame<T>::propagate does (src/Cell/PoolCell_Frame.cpp:123-175)
        checkStatus(n2d2hip_pool_average_f32_forward((int)mIn->dimB(), (int)mNbOutputs, (int)mInH, (int)mInW, (int)mPoolDims[0], (int)mPoolDims[1],
                                                     (int)mStrideDims[0], (int)mStrideDims[1], (int)mPaddingDims[0], (int)mPaddingDims[1], 1,
                                                     mIn->data(), mOutputs.data(), mStream));
    activationPropagate(inference);
    mDiffInputs.clearValid();
}

template <class T>
void PoolCell_FrameTrain_HIP<T>::backPropagate()
{
    if (!mDiffInputs.isValid())
        return;
    activationBackPropagate();
    if (!mDiffOut || mDiffOut->empty())
        return;
    const float beta = mDiffOut->isValid() ? 1.0f : 0.0f;
    if (mPooling == Max)
        checkStatus(n2d2hip_pool_max_f32_backward((int)mIn->dimB(), (int)mNbOutputs, (int)mInH, (int)mInW, (int)mPoolDims[0], (int)mPoolDims[1],
                                                  (int)mStrideDims[0], (int)mStrideDims[1], (int)mPaddingDims[0], (int)mPaddingDims[1],
                                                  mDiffInputs.data(), mArgMax, beta, mDiffOut->data(), mStream));
    else
        checkStatus(n2d2hip_pool_average_f32_backward((int)mIn->dimB(), (int)mNbOutputs, (int)mInH, (int)mInW, (int)mPoolDims[0], (int)mPoolDims[1],
                                                      (int)mStrideDims[0], (int)mStrideDims[1], (int)mPaddingDims[0], (int)mPaddingDims[1], 1,
                                                      mDiffInputs.data(), beta, mDiffOut->data(), mStream));
    mDiffOut->setValid();
}

template class PoolCell_FrameTrain_HIP<float>;
template <> Registrar<PoolCell> PoolCell_FrameTrain_HIP<float>::mRegistrar("Frame_HIP_QAT", PoolCell_FrameTrain_HIP<float>::create,
                                                                           Registrar<PoolCell>::Type<float>());

// -------------------------------------------------- ElemWiseCell_FrameTrain_HIP
ElemWiseCell_FrameTrain_HIP::ElemWiseCell_FrameTrain_HIP(const DeepNet& /*deepNet*/, const std::string& name, unsigned int nbOutputs,
                                                         Operation operation, CoeffMode mode, const std::vector<Float_T>& weights,
                                                         const std::vector<Float_T>& shifts, const std::shared_ptr<Activation>& activation)
    : Cell(name, nbOutputs), ElemWiseCell(operation, mode, weights, shifts)
{
    if (operation != Sum)
        throw std::runtime_error("ElemWiseCell_FrameTrain_HIP " + name + ": only Operation=Sum is supported by the float Frame_HIP cells");
    if (mode == PerChannel)
        throw std::runtime_error("ElemWiseCell_FrameTrain_HIP " + name + ": one coefficient per channel is not supported by the float Frame_HIP cells");
    mActivation = activation;
}

void ElemWiseCell_FrameTrain_HIP::addInput(Cell_FrameTrain_HIP* parent)
{
    if (!parent)
        throw std::runtime_error("Cell " + mName + ": null parent");
    addInput(parent->getOutputs(), parent->getDiffInputs());
    mParents.back() = parent;
}

void ElemWiseCell_FrameTrain_HIP::addInput(DeviceFloats& inputs, DeviceFloats& diffOutputs)
{
    if (mIns.empty()) {
        Cell_FrameTrain_HIP::addInput(inputs, diffOutputs);
    } else {
        if (inputs.dims() != mIns[0]->dims())
            throw std::runtime_error("ElemWiseCell_FrameTrain_HIP " + mName + ": inputs of different sizes");
        if (!diffOutputs.empty() && diffOutputs.dims() != inputs.dims())
            throw std::runtime_error("Cell " + mName + ": inputs and diffOutputs of different sizes");
        mParents.push_back(nullptr);
    }
    mIns.push_back(&inputs);
    mDiffOuts.push_back(&diffOutputs);
}

void ElemWiseCell_FrameTrain_HIP::initialize()
{
    if (mIns.empty() || mIns.size() > N2D2HIP_ELEMWISE_F32_MAX_INPUTS)
        throw std::runtime_error("ElemWiseCell_FrameTrain_HIP " + mName + ": 1 to 8 inputs expected");
    if (mNbChannels != mNbOutputs)
        throw std::runtime_error("ElemWiseCell_FrameTrain_HIP " + mName + ": the number of outputs must be the number of input channels");
    // src/Cell/ElemWiseCell_Frame.cpp:75-87: weights 1 and shifts 0 where none are given, one entry per input (one for all
    // inputs is repeated)
    const size_t n = mIns.size();
    if (mWeights.empty()) mWeights.assign(n, 1.0f);
    if (mShifts.empty()) mShifts.assign(n, 0.0f);
    if (mWeights.size() == 1) mWeights.assign(n, mWeights[0]);
    if (mShifts.size() == 1) mShifts.assign(n, mShifts[0]);
    if (mWeights.size() != n || mShifts.size() != n)
        throw std::runtime_error("ElemWiseCell_FrameTrain_HIP " + mName + ": one weight and one shift per input expected");
    allocateOutputs();
}

void ElemWiseCell_FrameTrain_HIP::propagate(bool inference)
{
    std::vector<const float*> ins;
    for (const DeviceFloats* t : mIns)
        ins.push_back(t->data());
    checkStatus(n2d2hip_elemwise_sum_f32_forward((int)ins.size(), ins.data(), mOutputs.size(), mWeights.data(), mShifts.data(), mOutputs.data(),
                                                 mStream));
    activationPropagate(inference);
    mDiffInputs.clearValid();
}

void ElemWiseCell_FrameTrain_HIP::backPropagate()
{
    if (!mDiffInputs.isValid())
        return;
    activationBackPropagate();
    for (size_t k = 0; k < mIns.size(); ++k) {
        DeviceFloats* d = mDiffOuts[k];
        if (!d || d->empty())
            continue;
        checkStatus(n2d2hip_elemwise_sum_f32_backward(mDiffInputs.size(), mWeights[k], mDiffInputs.data(), d->isValid() ? 1.0f : 0.0f, d->data(),
                                                      mStream));
        d->setValid();
    }
}

Registrar<ElemWiseCell> ElemWiseCell_FrameTrain_HIP::mRegistrar("Frame_HIP_QAT", ElemWiseCell_FrameTrain_HIP::create,
                                                                Registrar<ElemWiseCell>::Type<float>());

// --------------------------------------------------- SoftmaxCell_FrameTrain_HIP
const char* SoftmaxCell::Type = "Softmax";

template <class T>
SoftmaxCell_FrameTrain_HIP<T>::SoftmaxCell_FrameTrain_HIP(const DeepNet& /*deepNet*/, const std::string& name, unsigned int nbOutputs, bool withLoss,
                                                          unsigned int groupSize)
    : Cell(name, nbOutputs), SoftmaxCell(withLoss, groupSize)
{
    if (groupSize != 0 && groupSize != nbOutputs)
        throw std::runtime_error("SoftmaxCell_FrameTrain_HIP " + name + ": GroupSize is not supported by the float Frame_HIP cells");
}

template <class T>
void SoftmaxCell_FrameTrain_HIP<T>::initialize()
{
    if (mNbChannels != mNbOutputs)
        throw std::runtime_error("SoftmaxCell_FrameTrain_HIP " + mName + ": the number of outputs must be the number of input channels");
    allocateOutputs();
}

template <class T>
void SoftmaxCell_FrameTrain_HIP<T>::propagate(bool /*inference*/)
{
    checkStatus(n2d2hip_softmax_f32_forward(mIn->data(), mOutputs.data(), (int)mIn->dimB(), (int)mNbOutputs, (int)mOutH, (int)mOutW, mStream));
    mDiffInputs.clearValid();
}

template <class T>
void SoftmaxCell_FrameTrain_HIP<T>::backPropagate()
{
    if (!mDiffOut || mDiffOut->empty() || !mDiffInputs.isValid())
        return;
    if (!mWithLoss)
        throw std::runtime_error("SoftmaxCell_FrameTrain_HIP " + mName + ": backPropagate() without WithLoss is not supported by the float Frame_HIP cells");
    if (mDiffOut->isValid())       // another consumer of the input has written its part: add to it
        checkStatus(n2d2hip_elemwise_sum_f32_backward(mDiffInputs.size(), 1.0f, mDiffInputs.data(), 1.0f, mDiffOut->data(), mStream));
    else
        checkHipT(hipMemcpyAsync(mDiffOut->data(), mDiffInputs.data(), mDiffInputs.size() * sizeof(float), hipMemcpyDeviceToDevice, (hipStream_t)mStream),
                  "SoftmaxCell_FrameTrain_HIP::backPropagate()");
    mDiffOut->setValid();
}

template class SoftmaxCell_FrameTrain_HIP<float>;
template <> Registrar<SoftmaxCell> SoftmaxCell_FrameTrain_HIP<float>::mRegistrar("Frame_HIP_QAT", SoftmaxCell_FrameTrain_HIP<float>::create,
                                                                                 Registrar<SoftmaxCell>::Type<float>());

} // namespace N2D2
