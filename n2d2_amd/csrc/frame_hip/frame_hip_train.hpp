// Float cells of the Frame_HIP model for quantization-aware training: the cells a SAT / LSQ graph learns with
// (convolution with a weight quantizer, activation with an activation quantizer, softmax with loss), device resident,
// with propagate / backPropagate / update as the reference's Frame cells have them.  Tensors are N2D2's own float
// tensors ({X,Y,Z,B}, X fastest) held in device memory; every computation goes through the C ABI (n2d2hip.h).
//
// These cells are registered under the model key "Frame_HIP_QAT": the key "Frame_HIP" holds the integer inference
// cells, which have the same cell types and the same element type (float) in the Registrar.
#ifndef N2D2_FRAME_HIP_TRAIN_HPP
#define N2D2_FRAME_HIP_TRAIN_HPP

#include "frame_hip.hpp"

namespace N2D2 {

// Device float tensor with N2D2's dimension order and the "valid" flag the reference keeps on gradient tensors
// (BaseTensor::isValid / setValid / clearValid, include/containers/Tensor.hpp:137-139).
class DeviceFloats {
public:
    DeviceFloats() : mData(nullptr), mDims{0, 0, 0, 0}, mValid(false) {}
    ~DeviceFloats();
    DeviceFloats(const DeviceFloats&) = delete;
    DeviceFloats& operator=(const DeviceFloats&) = delete;
    void resize(const std::vector<size_t>& dims);        // zero-filled
    bool empty() const { return mData == nullptr; }
    size_t dimX() const { return mDims[0]; }
    size_t dimY() const { return mDims[1]; }
    size_t dimZ() const { return mDims[2]; }
    size_t dimB() const { return mDims[3]; }
    const std::vector<size_t>& dims() const { return mDims; }
    size_t size() const { return mDims[0] * mDims[1] * mDims[2] * mDims[3]; }
    float* data() { return mData; }
    const float* data() const { return mData; }
    bool isValid() const { return mValid; }
    void setValid() { mValid = true; }
    void clearValid() { mValid = false; }
    void fromHost(const Tensor<Float_T>& host);
    void fromHost(const float* host, size_t n);
    Tensor<Float_T> toHost() const;

private:
    float* mData;
    std::vector<size_t> mDims;
    bool mValid;
};

// Common part of the float cells (the role of Cell_Frame<T>, src/Cell/Cell_Frame.cpp:100-160 and :474-492): one input
// tensor and the tensor its gradient goes to, own outputs and the gradient with respect to them, the activation
// applied in place.
class Cell_FrameTrain_HIP : public virtual Cell {
public:
    // Cell::addInput(Cell*): input = the parent's outputs, diffOutputs = the parent's diffInputs
    virtual void addInput(Cell_FrameTrain_HIP* parent);
    // Cell_Frame<T>::addInput(BaseTensor& inputs, BaseTensor& diffOutputs): an empty diffOutputs stops the gradient here
    virtual void addInput(DeviceFloats& inputs, DeviceFloats& diffOutputs);
    virtual void initialize() = 0;
    virtual void propagate(bool inference = false) = 0;
    virtual void backPropagate() = 0;
    virtual void update() = 0;
    DeviceFloats& getOutputs() { return mOutputs; }
    DeviceFloats& getDiffInputs() { return mDiffInputs; }
    // Cell_Frame<T>::applyLoss() (src/Cell/Cell_Frame.cpp:646-650 over Cell_Frame_Top::applyLoss,
    // src/Cell/Cell_Frame_Top.cpp:27-40): diffInputs, holding the targets, becomes targets - outputs; returns the sum of
    // squares over the batch size
    double applyLoss();
    bool isCuda() const { return false; }
    std::string getPyModel() const { return "Frame_HIP_QAT"; }
    // The stream this cell's kernels are launched on: whatever a caller copies into the cell's tensors between two of its
    // passes goes to the same stream, so that the order does not depend on a stream's implicit synchronisation.
    void* stream() const { return mStream; }

protected:
    Cell_FrameTrain_HIP() : mIn(nullptr), mDiffOut(nullptr), mStream(nullptr), mLoss(nullptr), mLossWorkspace(nullptr), mLossWorkspaceBytes(0) {}
    ~Cell_FrameTrain_HIP();
    virtual void setOutputsDims() = 0;
    void allocateOutputs();
    // Cell_Frame<T>::propagate / backPropagate / update: the activation in place on mOutputs / mDiffInputs
    void activationPropagate(bool inference);
    void activationBackPropagate();
    void activationUpdate();
    DeviceFloats* mIn;
    DeviceFloats* mDiffOut;
    DeviceFloats mOutputs, mDiffInputs;
    void* mStream;                  // the default stream: the quantizers attached to a cell launch there too

private:
    double* mLoss;
    void* mLossWorkspace;
    size_t mLossWorkspaceBytes;
};

// What ConvCell_Frame and FcCell_Frame share when they learn: device weights and biases with their gradients, the weight
// quantizer, the solvers, and the three convolution passes (an FcCell is the convolution whose kernel spans its input).
class WeightedCell_FrameTrain_HIP : public Cell_FrameTrain_HIP {
public:
    // Cell::setQuantizer (include/Cell/Cell.hpp:455-463), before initialize()
    void setQuantizer(const std::shared_ptr<QuantizerCell>& quantizer) { mQuantizer = quantizer; }
    const std::shared_ptr<QuantizerCell>& getQuantizer() const { return mQuantizer; }
    void setWeightsSolver(const std::shared_ptr<SGDSolver>& solver) { mWeightsSolver = solver; }
    void setBiasSolver(const std::shared_ptr<SGDSolver>& solver) { mBiasSolver = solver; }
    Tensor<Float_T> getDiffWeights() const { return mDevDiffW.toHost(); }
    Tensor<Float_T> getQuantizedWeights() const;
    // What DeepNetQAT reads of this cell once it has propagated: the weight quantizer's tensor (the weights themselves
    // without one), the biases, the quantizer's range, mode and SAT divisor
    QATCellParameters getQATCellParameters();
    // refreshes the host tensors getWeights() / getBiases() return from the device
    virtual void synchronizeWeightsToHost() = 0;

protected:
    WeightedCell_FrameTrain_HIP();
    virtual n2d2hip_conv_desc desc() const = 0;
    // uploads weights (dims as the cell holds them) and biases, allocates the gradients, hands the weights to the quantizer
    void initializeWeights(const Tensor<Float_T>& weights, Tensor<Float_T>& biases, bool noBias, size_t quantizerOutputsSize);
    void propagateWeighted(bool inference, bool noBias);
    void backPropagateWeighted(bool noBias);
    void updateWeighted(bool noBias);
    std::shared_ptr<QuantizerCell> mQuantizer;
    std::shared_ptr<SGDSolver> mWeightsSolver, mBiasSolver;
    DeviceFloats mDevW, mDevDiffW, mDevBias, mDevDiffBias;
    DeviceFloats mWorkspace;        // partial sums of the convolution passes
};

// src/Cell/ConvCell_Frame.cpp:418-597 for one input tensor.
template <class T>
class ConvCell_FrameTrain_HIP : public ConvCell, public WeightedCell_FrameTrain_HIP {
public:
    ConvCell_FrameTrain_HIP(const DeepNet& deepNet, const std::string& name, const std::vector<unsigned int>& kernelDims,
                            unsigned int nbOutputs, const std::vector<unsigned int>& subSampleDims,
                            const std::vector<unsigned int>& strideDims, const std::vector<int>& paddingDims,
                            const std::vector<unsigned int>& dilationDims, const std::shared_ptr<Activation>& activation);
    ~ConvCell_FrameTrain_HIP();
    static std::shared_ptr<ConvCell> create(Network& /*net*/, const DeepNet& deepNet, const std::string& name,
                                            const std::vector<unsigned int>& kernelDims, unsigned int nbOutputs,
                                            const std::vector<unsigned int>& subSampleDims, const std::vector<unsigned int>& strideDims,
                                            const std::vector<int>& paddingDims, const std::vector<unsigned int>& dilationDims,
                                            const std::shared_ptr<Activation>& activation)
    {
        return std::make_shared<ConvCell_FrameTrain_HIP<T> >(deepNet, name, kernelDims, nbOutputs, subSampleDims, strideDims,
                                                             paddingDims, dilationDims, activation);
    }
    // uploads the host weights / biases (ConvCell::setWeights, {kW, kH, C/groups, O}) before anything else
    void initialize();
    void propagate(bool inference = false) { propagateWeighted(inference, mNoBias); }
    void backPropagate() { backPropagateWeighted(mNoBias); }
    void update() { updateWeighted(mNoBias); }
    void synchronizeWeightsToHost();

protected:
    void setOutputsDims();
    n2d2hip_conv_desc desc() const;

private:
    static Registrar<ConvCell> mRegistrar;
};

// src/Cell/FcCell_Frame.cpp:234-480 for one input tensor: weights {K, O} with K = C*H*W in CHW order.
template <class T>
class FcCell_FrameTrain_HIP : public FcCell, public WeightedCell_FrameTrain_HIP {
public:
    FcCell_FrameTrain_HIP(const DeepNet& deepNet, const std::string& name, unsigned int nbOutputs, const std::shared_ptr<Activation>& activation);
    static std::shared_ptr<FcCell> create(Network& /*net*/, const DeepNet& deepNet, const std::string& name, unsigned int nbOutputs,
                                          const std::shared_ptr<Activation>& activation)
    {
        return std::make_shared<FcCell_FrameTrain_HIP<T> >(deepNet, name, nbOutputs, activation);
    }
    void initialize();
    void propagate(bool inference = false) { propagateWeighted(inference, mNoBias); }
    void backPropagate() { backPropagateWeighted(mNoBias); }
    void update() { updateWeighted(mNoBias); }
    void synchronizeWeightsToHost();

protected:
    void setOutputsDims() { mOutW = 1; mOutH = 1; }
    n2d2hip_conv_desc desc() const;

private:
    static Registrar<FcCell> mRegistrar;
};

// include/Cell/ActivationCell.hpp:36-60
class ActivationCell : public virtual Cell {
public:
    typedef std::function<std::shared_ptr<ActivationCell>(const DeepNet&, const std::string&, unsigned int,
                                                          const std::shared_ptr<Activation>&)> RegistryCreate_T;
    static RegistryMap_T& registry() { static RegistryMap_T rMap; return rMap; }
    static const char* Type;
    const char* getType() const { return Type; }
};

// src/Cell/ActivationCell_Frame.cpp:95-205 for one input: copy, then the activation in place.
template <class T>
class ActivationCell_FrameTrain_HIP : public ActivationCell, public Cell_FrameTrain_HIP {
public:
    ActivationCell_FrameTrain_HIP(const DeepNet& deepNet, const std::string& name, unsigned int nbOutputs,
                                  const std::shared_ptr<Activation>& activation);
    static std::shared_ptr<ActivationCell> create(const DeepNet& deepNet, const std::string& name, unsigned int nbOutputs,
                                                  const std::shared_ptr<Activation>& activation)
    {
        return std::make_shared<ActivationCell_FrameTrain_HIP<T> >(deepNet, name, nbOutputs, activation);
    }
    void initialize();
    void propagate(bool inference = false);
    void backPropagate();
    void update() { activationUpdate(); }

protected:
    void setOutputsDims() { mOutW = mInW; mOutH = mInH; }

private:
    static Registrar<ActivationCell> mRegistrar;
};

// include/Cell/BatchNormCell.hpp:36-160: Epsilon (1.0e-5), MovingAverageMomentum (0.1); scales 1, biases 0, means 0,
// variances 0 until set or learned
class BatchNormCell : public virtual Cell {
public:
    typedef std::function<std::shared_ptr<BatchNormCell>(const DeepNet&, const std::string&, unsigned int,
                                                         const std::shared_ptr<Activation>&)> RegistryCreate_T;
    static RegistryMap_T& registry() { static RegistryMap_T rMap; return rMap; }
    static const char* Type;
    const char* getType() const { return Type; }
    void setParameter(const std::string& name, double value);
    double getEpsilon() const { return mEpsilon; }

protected:
    BatchNormCell() : mEpsilon(1.0e-5), mMovingAverageMomentum(0.1) {}
    double mEpsilon, mMovingAverageMomentum;
};

// src/Cell/BatchNormCell_Frame.cpp for one input.  Parameters, statistics and gradients stay on the device; the
// getters copy to the host, the setters (before or after initialize()) to the device.
template <class T>
class BatchNormCell_FrameTrain_HIP : public BatchNormCell, public Cell_FrameTrain_HIP {
public:
    BatchNormCell_FrameTrain_HIP(const DeepNet& deepNet, const std::string& name, unsigned int nbOutputs,
                                 const std::shared_ptr<Activation>& activation);
    static std::shared_ptr<BatchNormCell> create(const DeepNet& deepNet, const std::string& name, unsigned int nbOutputs,
                                                 const std::shared_ptr<Activation>& activation)
    {
        return std::make_shared<BatchNormCell_FrameTrain_HIP<T> >(deepNet, name, nbOutputs, activation);
    }
    void initialize();
    void propagate(bool inference = false);
    void backPropagate();
    void update();
    // BatchNormCell::setScales / setBiases / setMeans / setVariances and their getters, one value per output
    void setScales(const std::vector<Float_T>& v) { set(mScale, mHostScale, v); }
    void setBiases(const std::vector<Float_T>& v) { set(mBias, mHostBias, v); }
    void setMeans(const std::vector<Float_T>& v) { set(mMean, mHostMean, v); }
    void setVariances(const std::vector<Float_T>& v) { set(mVariance, mHostVariance, v); }
    std::vector<Float_T> getScales() const { return get(mScale, mHostScale); }
    std::vector<Float_T> getBiases() const { return get(mBias, mHostBias); }
    std::vector<Float_T> getMeans() const { return get(mMean, mHostMean); }
    std::vector<Float_T> getVariances() const { return get(mVariance, mHostVariance); }
    std::vector<Float_T> getDiffScales() const { return get(mDiffScale, std::vector<Float_T>()); }
    std::vector<Float_T> getDiffBiases() const { return get(mDiffBias, std::vector<Float_T>()); }
    void setScaleSolver(const std::shared_ptr<SGDSolver>& solver) { mScaleSolver = solver; }
    void setBiasSolver(const std::shared_ptr<SGDSolver>& solver) { mBiasSolver = solver; }
    const std::shared_ptr<SGDSolver>& getScaleSolver() const { return mScaleSolver; }
    const std::shared_ptr<SGDSolver>& getBiasSolver() const { return mBiasSolver; }
    // What DeepNetQAT reads of this cell: the four vectors, Epsilon, and range and alpha of the SAT quantizer of its
    // activation (range 0 without one)
    BatchNormParameters getBatchNormParameters() const;

protected:
    void setOutputsDims() { mOutW = mInW; mOutH = mInH; }

private:
    void set(DeviceFloats& dev, std::vector<Float_T>& host, const std::vector<Float_T>& v);
    std::vector<Float_T> get(const DeviceFloats& dev, const std::vector<Float_T>& host) const;
    DeviceFloats mScale, mBias, mMean, mVariance, mSavedMean, mSavedVariance, mDiffScale, mDiffBias, mDiffSavedMean, mDiffSavedVariance;
    DeviceFloats mDiffOwn;      // this cell's part of the input gradient while another consumer's is already there
    DeviceFloats mWorkspace;            // partial sums of the split reductions
    std::vector<Float_T> mHostScale, mHostBias, mHostMean, mHostVariance;      // values set before initialize()
    std::shared_ptr<SGDSolver> mScaleSolver, mBiasSolver;
    bool mLearned;              // a learning propagate has filled the saved statistics
    static Registrar<BatchNormCell> mRegistrar;
};

// src/Cell/PoolCell_Frame.cpp:123-228 with Pooling=Max or Average (padding counted), one input and one output per channel.
template <class T>
class PoolCell_FrameTrain_HIP : public PoolCell, public Cell_FrameTrain_HIP {
public:
    PoolCell_FrameTrain_HIP(const DeepNet& deepNet, const std::string& name, const std::vector<unsigned int>& poolDims, unsigned int nbOutputs,
                            const std::vector<unsigned int>& strideDims, const std::vector<unsigned int>& paddingDims, Pooling pooling,
                            const std::shared_ptr<Activation>& activation);
    ~PoolCell_FrameTrain_HIP();
    static std::shared_ptr<PoolCell> create(Network& /*net*/, const DeepNet& deepNet, const std::string& name,
                                            const std::vector<unsigned int>& poolDims, unsigned int nbOutputs,
                                            const std::vector<unsigned int>& strideDims, const std::vector<unsigned int>& paddingDims,
                                            Pooling pooling, const std::shared_ptr<Activation>& activation)
    {
        return std::make_shared<PoolCell_FrameTrain_HIP<T> >(deepNet, name, poolDims, nbOutputs, strideDims, paddingDims, pooling, activation);
    }
    void initialize();
    void propagate(bool inference = false);
    void backPropagate();
    void update() { activationUpdate(); }

protected:
    void setOutputsDims();

private:
    int* mArgMax;
    static Registrar<PoolCell> mRegistrar;
};

// src/Cell/ElemWiseCell_Frame.cpp:104-136 and :194-233, Operation Sum with one coefficient per input (or one for all):
// outputs = (w0 x0 + s0) + (w1 x1 + s1) + ..., the gradient towards input k = wk times the gradient of the outputs, added
// to what another consumer of that input has already written.  The cell of a residual sum in a learning graph.
class ElemWiseCell_FrameTrain_HIP : public ElemWiseCell, public Cell_FrameTrain_HIP {
public:
    ElemWiseCell_FrameTrain_HIP(const DeepNet& deepNet, const std::string& name, unsigned int nbOutputs, Operation operation, CoeffMode mode,
                                const std::vector<Float_T>& weights, const std::vector<Float_T>& shifts,
                                const std::shared_ptr<Activation>& activation);
    static std::shared_ptr<ElemWiseCell> create(Network& /*net*/, const DeepNet& deepNet, const std::string& name, unsigned int nbOutputs,
                                                Operation operation, CoeffMode mode, const std::vector<Float_T>& weights,
                                                const std::vector<Float_T>& shifts, const std::shared_ptr<Activation>& activation)
    {
        return std::make_shared<ElemWiseCell_FrameTrain_HIP>(deepNet, name, nbOutputs, operation, mode, weights, shifts, activation);
    }
    // every input has the size of the first one
    void addInput(Cell_FrameTrain_HIP* parent);
    void addInput(DeviceFloats& inputs, DeviceFloats& diffOutputs);
    void initialize();
    void propagate(bool inference = false);
    void backPropagate();
    void update() { activationUpdate(); }

protected:
    void setOutputsDims() { mOutW = mInW; mOutH = mInH; }

private:
    std::vector<DeviceFloats*> mIns, mDiffOuts;
    static Registrar<ElemWiseCell> mRegistrar;
};

// include/Cell/SoftmaxCell.hpp:37-70: WithLoss (false), GroupSize (0)
class SoftmaxCell : public virtual Cell {
public:
    typedef std::function<std::shared_ptr<SoftmaxCell>(const DeepNet&, const std::string&, unsigned int, bool, unsigned int)> RegistryCreate_T;
    static RegistryMap_T& registry() { static RegistryMap_T rMap; return rMap; }
    static const char* Type;
    const char* getType() const { return Type; }

protected:
    SoftmaxCell(bool withLoss, unsigned int groupSize) : mWithLoss(withLoss), mGroupSize(groupSize) {}
    bool mWithLoss;
    unsigned int mGroupSize;
};

// src/Cell/SoftmaxCell_Frame.cpp:93-207, one group, WithLoss (the gradient of the loss passes through unchanged).
template <class T>
class SoftmaxCell_FrameTrain_HIP : public SoftmaxCell, public Cell_FrameTrain_HIP {
public:
    SoftmaxCell_FrameTrain_HIP(const DeepNet& deepNet, const std::string& name, unsigned int nbOutputs, bool withLoss = false,
                               unsigned int groupSize = 0);
    static std::shared_ptr<SoftmaxCell> create(const DeepNet& deepNet, const std::string& name, unsigned int nbOutputs, bool withLoss,
                                               unsigned int groupSize)
    {
        return std::make_shared<SoftmaxCell_FrameTrain_HIP<T> >(deepNet, name, nbOutputs, withLoss, groupSize);
    }
    void initialize();
    void propagate(bool inference = false);
    void backPropagate();
    void update() {}

protected:
    void setOutputsDims() { mOutW = mInW; mOutH = mInH; }

private:
    static Registrar<SoftmaxCell> mRegistrar;
};

} // namespace N2D2

#endif
