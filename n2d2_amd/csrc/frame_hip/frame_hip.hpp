// Host side of the "Frame_HIP" model: C++ cells that plug into N2D2's Registrar
// under the key "Frame_HIP" and drive the HIP kernels through the C ABI of
// n2d2hip.h.  The classes mirror the N2D2 interfaces they stand in for (same
// names, constructor / factory signatures, parameter names and error behaviour);
// each cites the reference header it follows (paths relative to the N2D2 tree).
//
// This file also carries the small amount of N2D2 infrastructure the cells need
// to run without an N2D2 checkout (Registrar, Tensor, Scaling, a layer-ordered
// DeepNet): in an N2D2 build those come from N2D2's own headers and only the
// *_Frame_HIP classes and their registrations are compiled in (N2D2_EXTRAMODULE).
#pragma once

#include <cmath>
#include <cstdint>
#include <functional>
#include <iostream>
#include <limits>
#include <map>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <typeindex>
#include <utility>
#include <vector>

#include "n2d2hip.h"

namespace N2D2 {

typedef float Float_T;

// ------------------------------------------------------------------ Registrar
// Semantics of include/utils/Registrar.hpp:46-149: a static object whose constructor files a
// factory under (key, type); a duplicate (key, type) throws; an unknown key or type prints a
// message and yields an empty function.
struct BaseCommand {
    virtual ~BaseCommand() {}
};
typedef std::map<std::string, std::map<std::type_index, std::unique_ptr<BaseCommand> > > RegistryMap_T;

template <typename C, typename F = typename C::RegistryCreate_T>
struct Registrar {
    struct Command : public BaseCommand {
        F mFunc;
        explicit Command(F func) : mFunc(func) {}
    };
    template <class T>
    struct Type {};

    template <class T = void>
    Registrar(const std::string& key, F func, const Type<T>& = Type<T>())
    {
        auto& perType = C::registry()[key];
        const std::type_index idx(typeid(T));
        if (perType.count(idx))
            throw std::runtime_error("Registrar \"" + key + "\" already exists");
        perType[idx].reset(new Command(func));
    }
    static bool exists(const std::string& key) { return C::registry().count(key) != 0; }
    template <class T>
    static bool exists(const std::string& key)
    {
        auto it = C::registry().find(key);
        return it != C::registry().end() && it->second.count(std::type_index(typeid(T))) != 0;
    }
    template <class T = void>
    static F create(const std::string& key)
    {
        auto it = C::registry().find(key);
        if (it == C::registry().end()) {
            std::cout << "Invalid registrar key \"" << key << "\"" << std::endl;
            return F();
        }
        auto itType = it->second.find(std::type_index(typeid(T)));
        if (itType == it->second.end()) {
            std::cout << "Invalid registrar key type (" << typeid(T).name() << ") for key \"" << key << "\"" << std::endl;
            return F();
        }
        return static_cast<Command*>(itType->second.get())->mFunc;
    }
};

// --------------------------------------------------------------------- Tensor
// Host tensor with N2D2's dimension order {X, Y, Z, B}, X fastest
// (include/containers/Tensor.hpp:162-193).
template <class T>
class Tensor {
public:
    Tensor() : mDims{0, 0, 0, 0} {}
    explicit Tensor(const std::vector<size_t>& dims, T value = T()) { resize(dims, value); }
    void resize(const std::vector<size_t>& dims, T value = T())
    {
        mDims = dims;
        while (mDims.size() < 4) mDims.push_back(1);
        mData.assign(size(), value);
    }
    size_t dimX() const { return mDims[0]; }
    size_t dimY() const { return mDims[1]; }
    size_t dimZ() const { return mDims[2]; }
    size_t dimB() const { return mDims[3]; }
    const std::vector<size_t>& dims() const { return mDims; }
    size_t size() const { return mDims[0] * mDims[1] * mDims[2] * mDims[3]; }
    bool empty() const { return mData.empty(); }
    T& operator()(size_t i) { return mData[i]; }
    const T& operator()(size_t i) const { return mData[i]; }
    T& operator()(size_t x, size_t y, size_t z, size_t b) { return mData[x + mDims[0] * (y + mDims[1] * (z + mDims[2] * b))]; }
    const T& operator()(size_t x, size_t y, size_t z, size_t b) const { return mData[x + mDims[0] * (y + mDims[1] * (z + mDims[2] * b))]; }
    T* data() { return mData.data(); }
    const T* data() const { return mData.data(); }
    // by value: also usable where T is bool
    T at(size_t x, size_t y) const { return mData[x + mDims[0] * y]; }
    void set(size_t x, size_t y, T v) { mData[x + mDims[0] * y] = v; }
    void fill(T v) { std::fill(mData.begin(), mData.end(), v); }

private:
    std::vector<size_t> mDims;
    std::vector<T> mData;
};

// Throws std::runtime_error carrying the library's message when a C-ABI call fails:
// the reference reports every error as a C++ exception.
void checkStatus(int status);

// Device tensor of a Frame_HIP cell: narrow integer storage in the private NHWC form,
// with a host float mirror refreshed on demand so that Frame cells, Targets or tests can
// still read N2D2-style float tensors (the role CudaTensor plays, include/containers/CudaTensor.hpp:256-359).
class HipTensor {
public:
    HipTensor() : mDesc(), mBytes(0), mHostValid(false) {}
    ~HipTensor();
    HipTensor(const HipTensor&) = delete;
    HipTensor& operator=(const HipTensor&) = delete;
    // halo: border pixels stored around every image, holding the value 0 (tensors between two convolutions).
    // stimuli: the network's input, which may use the 4-byte channel stride the first-layer kernel reads; what a cell
    // writes always has a stride that is a multiple of 16.
    void resize(int B, int C, int H, int W, int dtype, int halo = 0, bool stimuli = false);
    // The network's input in the space-to-depth form a first-layer convolution of stride 2 reads (N2D2HIP_S2D), with a
    // border of `halo` 16-byte pixels; synchronizeHToD() fills all of it.
    void resizeSpaceToDepth(int B, int C, int H, int W, int dtype, int halo);
    const n2d2hip_tensor& desc() const { return mDesc; }
    bool empty() const { return mDesc.data == nullptr; }
    void invalidateHost() { mHostValid = false; }
    // Integer-valued floats, NCHW / {W,H,C,B}
    const Tensor<Float_T>& synchronizeDToH(void* stream = nullptr);
    void synchronizeHToD(const Tensor<Float_T>& host, void* stream = nullptr);

private:
    n2d2hip_tensor mDesc;
    size_t mBytes;
    Tensor<Float_T> mHost;
    bool mHostValid;
};

// ---------------------------------------------------------------- ScalingMode
// include/ScalingMode.hpp:27-62
enum class ScalingMode { NONE, FLOAT_MULT, FIXED_MULT16, FIXED_MULT32, SINGLE_SHIFT, DOUBLE_SHIFT };
ScalingMode parseScalingMode(const std::string& str);

// -------------------------------------------------------------------- Scaling
// Value type with the factories and getters of include/Scaling.hpp:336-432.
class Scaling {
public:
    Scaling() : mMode(ScalingMode::NONE), mNbFractionalBits(0), mIsClipped(false) {}
    static Scaling floatingPointScaling(std::vector<Float_T> scalingPerOutput, bool isClipped, std::vector<Float_T> clippingPerOutput)
    {
        Scaling s;
        s.mMode = ScalingMode::FLOAT_MULT;
        s.mFloat = std::move(scalingPerOutput);
        s.mIsClipped = isClipped;
        s.mClipping = std::move(clippingPerOutput);
        return s;
    }
    static Scaling fixedPointScaling(ScalingMode mode, std::size_t nbFractionalBits, std::vector<std::int32_t> scalingPerOutput,
                                     bool isClipped, std::vector<Float_T> clippingPerOutput)
    {
        if (mode != ScalingMode::FIXED_MULT16 && mode != ScalingMode::FIXED_MULT32)
            throw std::runtime_error("Scaling::fixedPointScaling(): mode must be FIXED_MULT16 or FIXED_MULT32");
        Scaling s;
        s.mMode = mode;
        s.mNbFractionalBits = nbFractionalBits;
        s.mFixed = std::move(scalingPerOutput);
        s.mIsClipped = isClipped;
        s.mClipping = std::move(clippingPerOutput);
        return s;
    }
    static Scaling singleShiftScaling(std::vector<unsigned char> scalingPerOutput, bool isClipped, std::vector<Float_T> clippingPerOutput)
    {
        Scaling s;
        s.mMode = ScalingMode::SINGLE_SHIFT;
        s.mShift = std::move(scalingPerOutput);
        s.mIsClipped = isClipped;
        s.mClipping = std::move(clippingPerOutput);
        return s;
    }
    static Scaling doubleShiftScaling(std::vector<std::pair<unsigned char, unsigned char> > scalingPerOutput, bool isClipped,
                                      std::vector<std::pair<unsigned char, unsigned char> > /*clippingPerOutput*/)
    {
        Scaling s;
        s.mMode = ScalingMode::DOUBLE_SHIFT;
        for (const auto& p : scalingPerOutput) {
            s.mShift.push_back(p.first);
            s.mShift.push_back(p.second);
        }
        s.mIsClipped = isClipped;
        return s;
    }
    ScalingMode getMode() const { return mMode; }
    const std::vector<Float_T>& getFloatScalingPerOutput() const { return mFloat; }
    const std::vector<std::int32_t>& getFixedScalingPerOutput() const { return mFixed; }
    const std::vector<unsigned char>& getShiftScalingPerOutput() const { return mShift; }
    std::size_t getFractionalBits() const { return mNbFractionalBits; }
    bool getIsClipped() const { return mIsClipped; }
    const std::vector<Float_T>& getClippingPerOutput() const { return mClipping; }
    // Text form of everything this object holds (include/Scaling.hpp:336-432: mode, per-output factors, fractional bits,
    // clip flag and values), one "Key=values" line each; floats are written with the digits that read back to the same
    // bits.  N2D2 itself has no file format for a Scaling (Activation::save writes the parameters only,
    // src/Activation/Activation.cpp:66-97): this one carries a graph quantized in one process into another.
    void save(std::ostream& os) const;
    static Scaling load(std::istream& is, const std::string& what);
    // true when every factor is >= 0 (ScalingCell::getOutputsRange, src/Cell/ScalingCell.cpp:68-104)
    bool allScalingsPositive() const;
    std::size_t nbOutputs() const;

private:
    ScalingMode mMode;
    std::size_t mNbFractionalBits;
    std::vector<Float_T> mFloat;
    std::vector<std::int32_t> mFixed;
    std::vector<unsigned char> mShift;     // SINGLE_SHIFT: one per output; DOUBLE_SHIFT: {first, second} per output
    bool mIsClipped;
    std::vector<Float_T> mClipping;
};

class Cell;
class Cell_Frame_HIP;
class DeepNet;
class Network {};

// Static state that decides the saturation range (src/Export/DeepNetExport.cpp:370-388,
// set by calibNetwork, src/utils/Helper.cpp:670-673).
struct CellExport {
    static int mPrecision;
};
struct DeepNetExport {
    static bool mUnsignedData;
    static bool mEnvDataUnsigned;
    static bool isCellOutputUnsigned(const Cell& cell);
};

// ----------------------------------------------------------------- Activation
class QuantizerActivation;
// include/Activation/Activation.hpp:36-110
class Activation {
public:
    // Quantizer applied to the activation's output during quantization-aware training (Activation::setQuantizer,
    // include/Activation/Activation.hpp:84-92); read by the float cells only
    void setQuantizer(const std::shared_ptr<QuantizerActivation>& quantizer) { mQuantizer = quantizer; }
    const std::shared_ptr<QuantizerActivation>& getQuantizer() const { return mQuantizer; }
    virtual double clipping() const { return 0.0; }
    virtual ~Activation() {}
    virtual const char* getType() const = 0;
    virtual std::pair<double, double> getOutputRange() const = 0;
    const Scaling& getActivationScaling() const { return mScaling; }
    void setActivationScaling(Scaling scaling) { mScaling = std::move(scaling); ++mRevision; }
    void setQuantized(std::size_t nbBits) { mQuantizedNbBits = nbBits; ++mRevision; }
    std::size_t getQuantizedNbBits() const { return mQuantizedNbBits; }
    virtual void setParameter(const std::string& name, double value) = 0;
    unsigned revision() const { return mRevision; }
    // kind / leak for the C ABI
    virtual int abiKind() const = 0;
    virtual float leakSlope() const { return 0.0f; }

protected:
    Activation() : mQuantizedNbBits(0), mRevision(0) {}
    Scaling mScaling;
    std::size_t mQuantizedNbBits;
    unsigned mRevision;
    std::shared_ptr<QuantizerActivation> mQuantizer;
};

// src/Activation/RectifierActivation.cpp:26-40 (LeakSlope 0.0, Clipping 0.0)
class RectifierActivation : public Activation {
public:
    typedef std::function<std::shared_ptr<RectifierActivation>()> RegistryCreate_T;
    static RegistryMap_T& registry() { static RegistryMap_T rMap; return rMap; }
    static const char* Type;
    RectifierActivation() : mLeakSlope(0.0), mClipping(0.0) {}
    const char* getType() const { return Type; }
    std::pair<double, double> getOutputRange() const
    {
        const double max = mClipping > 0.0 ? mClipping : std::numeric_limits<double>::infinity();
        return mLeakSlope > 0.0 ? std::make_pair(-max, max) : std::make_pair(0.0, max);
    }
    void setParameter(const std::string& name, double value);
    int abiKind() const { return N2D2HIP_ACT_RECTIFIER; }
    float leakSlope() const { return (float)mLeakSlope; }
    double clipping() const { return mClipping; }

protected:
    double mLeakSlope, mClipping;
};

// src/Activation/LinearActivation.cpp:24-25 (Clipping 0.0)
class LinearActivation : public Activation {
public:
    typedef std::function<std::shared_ptr<LinearActivation>()> RegistryCreate_T;
    static RegistryMap_T& registry() { static RegistryMap_T rMap; return rMap; }
    static const char* Type;
    LinearActivation() : mClipping(0.0) {}
    const char* getType() const { return Type; }
    std::pair<double, double> getOutputRange() const
    {
        const double inf = std::numeric_limits<double>::infinity();
        return mClipping > 0.0 ? std::make_pair(-mClipping, mClipping) : std::make_pair(-inf, inf);
    }
    void setParameter(const std::string& name, double value);
    int abiKind() const { return N2D2HIP_ACT_LINEAR; }
    double clipping() const { return mClipping; }

protected:
    double mClipping;
};

template <class T>
class RectifierActivation_Frame_HIP : public RectifierActivation {
public:
    static std::shared_ptr<RectifierActivation> create() { return std::make_shared<RectifierActivation_Frame_HIP<T> >(); }
private:
    static Registrar<RectifierActivation> mRegistrar;
};
template <class T>
class LinearActivation_Frame_HIP : public LinearActivation {
public:
    static std::shared_ptr<LinearActivation> create() { return std::make_shared<LinearActivation_Frame_HIP<T> >(); }
private:
    static Registrar<LinearActivation> mRegistrar;
};

// ----------------------------------------------------------------------- Cell
// The part of include/Cell/Cell.hpp + include/Cell/Cell_Frame_Top.hpp the quantized path uses.
class Cell {
public:
    virtual ~Cell() {}
    virtual const char* getType() const = 0;
    const std::string& getName() const { return mName; }
    unsigned int getNbOutputs() const { return mNbOutputs; }
    unsigned int getNbChannels() const { return mNbChannels; }
    unsigned int getChannelsWidth() const { return mInW; }
    unsigned int getChannelsHeight() const { return mInH; }
    unsigned int getOutputsWidth() const { return mOutW; }
    unsigned int getOutputsHeight() const { return mOutH; }
    void setQuantized(std::size_t nbBits) { mQuantizedNbBits = nbBits; }
    bool isQuantized() const { return mQuantizedNbBits > 0; }
    std::size_t getQuantizedNbBits() const { return mQuantizedNbBits; }
    const std::vector<Cell*>& getParentsCells() const { return mParents; }   // nullptr entry = the environment
    // Cell_Frame_Top::getOutputsRange, include/Cell/Cell_Frame_Top.hpp:118-121
    virtual std::pair<double, double> getOutputsRange() const
    {
        const double inf = std::numeric_limits<double>::infinity();
        return mActivation ? mActivation->getOutputRange() : std::make_pair(-inf, inf);
    }
    // Cell::getOutputsRangeParents, src/Cell/Cell.cpp:310-337
    std::pair<double, double> getOutputsRangeParents() const;
    // Number of groups of a connection map {outputs, channels} (Cell::getNbGroups, src/Cell/Cell.cpp:251-300): G when the map
    // is G equal blocks on the diagonal (output o of block g sees exactly the channels of block g), 0 when the first output
    // sees no leading channel.  Any other map is counted as the reference counts it by hand (getNbGroupsHandMade); `regular`,
    // if given, tells which of the two it was.
    static std::size_t getNbGroups(const Tensor<bool>& map, bool* regular = nullptr);
    // Cell::getNbGroupsHandMade (src/Cell/Cell.cpp:178-249): the number of connected sets of outputs and channels, counted
    // from the first output that has a connection; 0 for a map without any.  A later output without a connection, on
    // which the reference's loop does not end, is refused.
    static std::size_t getNbGroupsHandMade(const Tensor<bool>& map);
    const std::shared_ptr<Activation>& getActivation() const { return mActivation; }
    void setActivation(const std::shared_ptr<Activation>& activation) { mActivation = activation; }
    // Free parameters as text files, "<base>_weights<.ext>" and "<base>_biases<.ext>" (or one file holding both), the
    // format N2D2 exports after training or quantization (include/Cell/Cell.hpp:355-372)
    virtual void importFreeParameters(const std::string& fileName, bool ignoreNotExists = false) { (void)fileName; (void)ignoreNotExists; }
    virtual void exportFreeParameters(const std::string& fileName) const { (void)fileName; }
    // Applies func to every weight and the bias of one output (Cell::processFreeParametersPerOutput,
    // include/Cell/Cell.hpp:402-407)
    virtual void processFreeParametersPerOutput(const std::function<Float_T(Float_T)>& func, std::size_t output) { (void)func; (void)output; }

protected:
    Cell(const std::string& name, unsigned int nbOutputs)
        : mName(name), mNbOutputs(nbOutputs), mNbChannels(0), mInW(0), mInH(0), mOutW(0), mOutH(0), mQuantizedNbBits(0) {}
    // virtual base: only the most derived class runs the constructor above
    Cell() : mNbOutputs(0), mNbChannels(0), mInW(0), mInH(0), mOutW(0), mOutH(0), mQuantizedNbBits(0) {}
    std::string mName;
    unsigned int mNbOutputs, mNbChannels, mInW, mInH, mOutW, mOutH;
    std::size_t mQuantizedNbBits;
    std::vector<Cell*> mParents;
    std::shared_ptr<Activation> mActivation;
};

// Common part of the Frame_HIP cells (the role of Cell_Frame_CUDA<T>, include/Cell/Cell_Frame_CUDA.hpp:44-178).
class Cell_Frame_HIP : public virtual Cell {
public:
    // Connects a parent cell (Cell::addInput(Cell*), include/Cell/Cell.hpp:265) ...
    virtual void addInput(Cell_Frame_HIP* parent);
    // ... or the environment: an integer-valued tensor of nbChannels x height x width per batch item
    // (Cell::addInput(StimuliProvider&), include/Cell/Cell.hpp:208).
    virtual void addInput(HipTensor& stimuli, unsigned int nbChannels, unsigned int height, unsigned int width, unsigned int batchSize);
    // Cell_Frame<T>::clearInputs / replaceInput (src/Cell/Cell_Frame.cpp:215-270): graph surgery.  Device tensors are
    // sized at initialize(), so the new input's dimensions come from the cell that produces it when one is named
    // (newParent, whose output tensor newInputs must be), else from the tensor, which must then be allocated.
    void clearInputs();
    void replaceInput(HipTensor& oldInputs, HipTensor& newInputs, Cell_Frame_HIP* newParent = nullptr);
    virtual void initialize() {}
    virtual void propagate(bool inference = false) = 0;
    // The integer cells infer only: learning is what the float cells of the model "Frame_HIP_QAT" do.  These three
    // throw, so that a learning loop handed a Frame_HIP net stops with a message instead of leaving weights untouched.
    virtual void backPropagate();
    virtual void update();
    virtual void checkGradient(double epsilon, double maxError);
    // Index of the largest output of one batch item, the first one on a tie (Cell_Frame<T>::getMaxOutput,
    // src/Cell/Cell_Frame.cpp:747-752)
    unsigned int getMaxOutput(unsigned int batchPos = 0);
    // propagate() in two halves, for a runner that fuses cells: prepare() (re)builds the device handles a parameter
    // change invalidated and tells whether it rebuilt any; launch() enqueues the kernels.
    virtual bool prepare() { return false; }
    virtual void launch() { propagate(true); }
    // Outputs as N2D2 sees them: float tensor {W,H,C,B} holding integer values.  Throws for a cell whose work a
    // consumer has taken over (DeepNet::setFusion): its tensor is never written.
    const Tensor<Float_T>& getOutputs();
    // The cell that computes this one's result on the fly instead of reading its output, if any
    Cell_Frame_HIP* foldedInto() const { return mFoldedInto; }
    void setFoldedInto(Cell_Frame_HIP* consumer) { mFoldedInto = consumer; }
    const std::vector<Cell_Frame_HIP*>& parentCells() const { return mParentCells; }
    HipTensor* inputTensor(size_t k) const { return mInputs.at(k); }
    size_t nbInputs() const { return mInputs.size(); }
    // Device handles a consumer borrows when it folds this cell (null for cells that cannot be folded)
    virtual n2d2hip_act_t scalingHandle() const { return nullptr; }
    virtual n2d2hip_conv_t convHandle() const { return nullptr; }
    // Largest padding this cell applies to its input (0 for cells without one)
    virtual int maxPadding() const { return 0; }
    // Stores the outputs with a border of `halo` zero pixels around every image (see n2d2hip_tensor::halo)
    void setOutputsHalo(int halo);
    int outputsHalo() const { return mOutputsHalo; }
    HipTensor& getDeviceOutputs() { return mOutputs; }
    bool isCuda() const { return false; }
    std::string getPyModel() const { return "Frame_HIP"; }
    std::string getPyDataType() const { return "float"; }
    unsigned int batchSize() const { return mBatch; }
    void setStream(void* stream) { mStream = stream; }

protected:
    Cell_Frame_HIP() : mBatch(0), mStream(nullptr), mFoldedInto(nullptr), mOutputsHalo(0), mActHandle(nullptr), mActRevision(~0u), mActUnsigned(-1), mActGeneration(0) {}
    ~Cell_Frame_HIP();
    virtual void setOutputsDims() = 0;
    // (Re)builds the device tables of the activation when its Scaling, its bit width or the
    // signedness decision changed; cells without activation get a pass-through / Scaling-only table.
    // A further input of a cell whose channels are all its inputs' channels one behind the other (Conv, Fc): same size and
    // batch as the first one, and all of them cells.
    void addInputChannels(Cell_Frame_HIP* parent);
    // Checks that the inputs share one storage type (DeepNetExport::isCellInputsUnsigned, src/Export/DeepNetExport.cpp:298-317,
    // refuses parents of mixed signedness) and sizes the tensor their channels are gathered into.  Returns that type.
    int prepareGathered();
    // Gathers the inputs' channels (one launch) and returns the tensor the cell's kernel then reads.
    const n2d2hip_tensor& gatherInputs();
    HipTensor mGathered;
    n2d2hip_act_t activationHandle(const Scaling* standalone = nullptr);
    // Counts the handles activationHandle() has made.  A cell remembers the count its own device handle was built at:
    // the handle's address says nothing, a new one may be allocated where the one before it was.
    unsigned long activationGeneration() const { return mActGeneration; }
    int outputDType(const Scaling* standalone = nullptr) const;
    void allocateOutputs(const Scaling* standalone = nullptr);
    std::vector<HipTensor*> mInputs;
    std::vector<Cell_Frame_HIP*> mParentCells;  // null = the environment
    HipTensor mOutputs;
    unsigned int mBatch;
    void* mStream;
    Cell_Frame_HIP* mFoldedInto;
    int mOutputsHalo;

private:
    n2d2hip_act_t mActHandle;
    unsigned mActRevision;
    int mActUnsigned;
    unsigned long mActGeneration;
};

// ------------------------------------------------------------------- ConvCell
// include/Cell/ConvCell.hpp:41-252
class ConvCell : public virtual Cell {
public:
    typedef std::function<std::shared_ptr<ConvCell>(Network&, const DeepNet&, const std::string&, const std::vector<unsigned int>&,
                                                    unsigned int, const std::vector<unsigned int>&, const std::vector<unsigned int>&,
                                                    const std::vector<int>&, const std::vector<unsigned int>&,
                                                    const std::shared_ptr<Activation>&)> RegistryCreate_T;
    static RegistryMap_T& registry() { static RegistryMap_T rMap; return rMap; }
    static const char* Type;
    const char* getType() const { return Type; }
    void setParameter(const std::string& name, bool value);
    // Depthwise / grouped connection: the regular mapping Cell::getNbGroups recognises (src/Cell/Cell.cpp:251-300).
    void setNbGroups(unsigned int groups) { mNbGroups = groups; mIrregularMap = Tensor<bool>(); mDirty = true; }
    // The same from the connection map itself, {nbOutputs, nbChannels} (what Mapping.* sections of an INI expand to).  A
    // map that is not a set of equal groups is kept: the cell then convolves every output with its connected channels only
    // (ConvCell_Frame_Kernels::forward skips the others, src/Cell/ConvCell_Frame_Kernels.cpp:93-96), and its weights are
    // sized as the reference sizes them, {kW, kH, C / G, O} for G > 1 hand-counted groups (output o then uses slice n for its
    // n-th connected channel, `:97`), {kW, kH, C, O} otherwise (src/Cell/ConvCell_Frame.cpp:172-177).
    void setMapping(const Tensor<bool>& map);
    bool hasIrregularMapping() const { return !mIrregularMap.empty(); }
    // Weights as N2D2 holds them: float tensor {kW, kH, C/groups, O} with integer values; bias {O}.
    void setWeights(const Tensor<Float_T>& weights) { mWeights = weights; mDirty = true; }
    void setBiases(const Tensor<Float_T>& biases) { mBias = biases; mDirty = true; }
    // 4: weights are handed to the device nibble-packed (values must fit [-8,7])
    void setWeightsPrecision(int bits) { mWeightBits = bits; mDirty = true; }
    const Tensor<Float_T>& getWeights() const { return mWeights; }
    const Tensor<Float_T>& getBiases() const { return mBias; }
    // OCHW text: one line per output, the kernels of its connected channels one after the other, kernel x fastest
    // (src/Cell/ConvCell.cpp:299-353, 511-679)
    void importFreeParameters(const std::string& fileName, bool ignoreNotExists = false);
    void exportFreeParameters(const std::string& fileName) const;
    void processFreeParametersPerOutput(const std::function<Float_T(Float_T)>& func, std::size_t output);

protected:
    ConvCell(const std::vector<unsigned int>& kernelDims, const std::vector<unsigned int>& subSampleDims,
             const std::vector<unsigned int>& strideDims, const std::vector<int>& paddingDims,
             const std::vector<unsigned int>& dilationDims);
    std::vector<unsigned int> mKernelDims, mSubSampleDims, mStrideDims, mDilationDims;
    std::vector<int> mPaddingDims;
    bool mNoBias;
    unsigned int mNbGroups;
    int mWeightBits;
    Tensor<Float_T> mWeights, mBias;
    Tensor<bool> mIrregularMap;             // {nbOutputs, nbChannels}; empty: every connection, or mNbGroups equal groups
    bool mDirty;
    // Slices of the weights tensor per output (the third dimension the cell expects)
    unsigned int weightSlices() const { return hasIrregularMapping() && mNbGroups <= 1 ? mNbChannels : mNbChannels / mNbGroups; }
    // The weights of a cell with an irregular map as those of a full connection, {kW, kH, C, O}: zeros where there is none
    Tensor<Float_T> fullConnectionWeights() const;
    std::vector<std::size_t> connectedSlices(std::size_t output) const;
};

template <class T>
class ConvCell_Frame_HIP : public ConvCell, public Cell_Frame_HIP {
public:
    ConvCell_Frame_HIP(const DeepNet& deepNet, const std::string& name, const std::vector<unsigned int>& kernelDims,
                       unsigned int nbOutputs, const std::vector<unsigned int>& subSampleDims,
                       const std::vector<unsigned int>& strideDims, const std::vector<int>& paddingDims,
                       const std::vector<unsigned int>& dilationDims, const std::shared_ptr<Activation>& activation);
    ~ConvCell_Frame_HIP();
    static std::shared_ptr<ConvCell> create(Network& /*net*/, const DeepNet& deepNet, const std::string& name,
                                            const std::vector<unsigned int>& kernelDims, unsigned int nbOutputs,
                                            const std::vector<unsigned int>& subSampleDims, const std::vector<unsigned int>& strideDims,
                                            const std::vector<int>& paddingDims, const std::vector<unsigned int>& dilationDims,
                                            const std::shared_ptr<Activation>& activation)
    {
        return std::make_shared<ConvCell_Frame_HIP<T> >(deepNet, name, kernelDims, nbOutputs, subSampleDims, strideDims,
                                                        paddingDims, dilationDims, activation);
    }
    // Several inputs (ConvCell_Frame<T>::propagate, src/Cell/ConvCell_Frame.cpp:438-459, adds up one weighted sum per
    // input, each with its slice of the weights): the cell's channels are all inputs' channels one behind the other, its
    // weights {kW, kH, all channels / groups, nbOutputs}.  The inputs are gathered into one tensor by an extra launch and
    // the convolution reads that; such a cell takes no part in the graph-level fusions.
    void addInput(Cell_Frame_HIP* parent);
    using Cell_Frame_HIP::addInput;
    void initialize();
    void propagate(bool inference = false);
    bool prepare();
    void launch();
    n2d2hip_conv_t convHandle() const { return mConv; }
    int maxPadding() const { return std::max(mPaddingDims[0], mPaddingDims[1]); }
    // Graph-level fusion (DeepNet::planFusion): this 1x1 convolution computes the 3x3 depthwise convolution `depthwise`,
    // whose output it alone reads, in its own launch (n2d2hip_dw_pw_*); the depthwise cell is then not launched and its
    // output never written.  Taken where the device library accepts the pair and expects one launch to be faster than two
    // (n2d2hip_dw_pw_pays).
    bool fuseDepthwise(Cell_Frame_HIP* depthwise);
    void clearFusion();
    bool computesDepthwise() const { return mDwPw != nullptr; }

protected:
    void setOutputsDims();

private:
    n2d2hip_conv_t mConv;
    unsigned long mConvActGen;
    int mConvInDType;
    n2d2hip_dw_pw_t mDwPw;
    Cell_Frame_HIP* mFusedDw;
    static Registrar<ConvCell> mRegistrar;
};

// --------------------------------------------------------------------- FcCell
// include/Cell/FcCell.hpp:43-49
class FcCell : public virtual Cell {
public:
    typedef std::function<std::shared_ptr<FcCell>(Network&, const DeepNet&, const std::string&, unsigned int,
                                                  const std::shared_ptr<Activation>&)> RegistryCreate_T;
    static RegistryMap_T& registry() { static RegistryMap_T rMap; return rMap; }
    static const char* Type;
    const char* getType() const { return Type; }
    void setParameter(const std::string& name, bool value);
    // {K, O} float tensor (K = C*H*W in CHW order), bias {O}
    void setWeights(const Tensor<Float_T>& weights) { mWeights = weights; mDirty = true; }
    void setBiases(const Tensor<Float_T>& biases) { mBias = biases; mDirty = true; }
    const Tensor<Float_T>& getWeights() const { return mWeights; }
    const Tensor<Float_T>& getBiases() const { return mBias; }
    // OC text: one line per output, one weight per input in CHW order (src/Cell/FcCell.cpp:110-298)
    void importFreeParameters(const std::string& fileName, bool ignoreNotExists = false);
    void exportFreeParameters(const std::string& fileName) const;
    void processFreeParametersPerOutput(const std::function<Float_T(Float_T)>& func, std::size_t output);

protected:
    FcCell() : mNoBias(false), mDirty(true) {}
    bool mNoBias;
    Tensor<Float_T> mWeights, mBias;
    bool mDirty;
};

template <class T>
class FcCell_Frame_HIP : public FcCell, public Cell_Frame_HIP {
public:
    FcCell_Frame_HIP(const DeepNet& deepNet, const std::string& name, unsigned int nbOutputs, const std::shared_ptr<Activation>& activation);
    ~FcCell_Frame_HIP();
    static std::shared_ptr<FcCell> create(Network& /*net*/, const DeepNet& deepNet, const std::string& name, unsigned int nbOutputs,
                                          const std::shared_ptr<Activation>& activation)
    {
        return std::make_shared<FcCell_Frame_HIP<T> >(deepNet, name, nbOutputs, activation);
    }
    // Several inputs (FcCell_Frame<T>::propagate, src/Cell/FcCell_Frame.cpp:273-336): one inner product per input over its
    // own weights, added up, and the bias added once per input (`:309` seeds every input's product with it).  The inputs'
    // channels are gathered by one extra launch; the weights are {all inputs' values in CHW order, nbOutputs}.
    void addInput(Cell_Frame_HIP* parent);
    using Cell_Frame_HIP::addInput;
    void initialize();
    void propagate(bool inference = false);
    bool prepare();
    void launch();
    n2d2hip_fc_t fcHandle() const { return mFc; }
    // Graph-level fusion (DeepNet::planFusion): this cell ends a run of fully-connected cells, each read by the next
    // alone; `earlier` (one or two cells, first to last) are computed in this cell's launch and their outputs are never
    // stored.  Returns false, and changes nothing, where the device library declines the run.
    bool fuseChain(const std::vector<FcCell_Frame_HIP<T>*>& earlier);
    void clearFusion();
    size_t nbChained() const { return mChained.size(); }

protected:
    void setOutputsDims();

private:
    n2d2hip_fc_t mFc;
    unsigned long mFcActGen;
    size_t mFcNbInputs;
    int mFcInDType = -1;
    n2d2hip_fc_chain_t mChain = nullptr;
    std::vector<FcCell_Frame_HIP<T>*> mChained;
    static Registrar<FcCell> mRegistrar;
};

// ------------------------------------------------------------------- PoolCell
// include/Cell/PoolCell.hpp:47-55
class PoolCell : public virtual Cell {
public:
    enum Pooling { Max, Average };
    typedef std::function<std::shared_ptr<PoolCell>(Network&, const DeepNet&, const std::string&, const std::vector<unsigned int>&,
                                                    unsigned int, const std::vector<unsigned int>&, const std::vector<unsigned int>&,
                                                    Pooling, const std::shared_ptr<Activation>&)> RegistryCreate_T;
    static RegistryMap_T& registry() { static RegistryMap_T rMap; return rMap; }
    static const char* Type;
    const char* getType() const { return Type; }
    Pooling getPooling() const { return mPooling; }

protected:
    PoolCell(const std::vector<unsigned int>& poolDims, const std::vector<unsigned int>& strideDims,
             const std::vector<unsigned int>& paddingDims, Pooling pooling)
        : mPoolDims(poolDims), mStrideDims(strideDims), mPaddingDims(paddingDims), mPooling(pooling) {}
    std::vector<unsigned int> mPoolDims, mStrideDims, mPaddingDims;
    Pooling mPooling;
};

template <class T>
class PoolCell_Frame_HIP : public PoolCell, public Cell_Frame_HIP {
public:
    PoolCell_Frame_HIP(const DeepNet& deepNet, const std::string& name, const std::vector<unsigned int>& poolDims, unsigned int nbOutputs,
                       const std::vector<unsigned int>& strideDims, const std::vector<unsigned int>& paddingDims, Pooling pooling,
                       const std::shared_ptr<Activation>& activation);
    static std::shared_ptr<PoolCell> create(Network& /*net*/, const DeepNet& deepNet, const std::string& name,
                                            const std::vector<unsigned int>& poolDims, unsigned int nbOutputs,
                                            const std::vector<unsigned int>& strideDims, const std::vector<unsigned int>& paddingDims,
                                            Pooling pooling, const std::shared_ptr<Activation>& activation)
    {
        return std::make_shared<PoolCell_Frame_HIP<T> >(deepNet, name, poolDims, nbOutputs, strideDims, paddingDims, pooling, activation);
    }
    // Several inputs (PoolCell_Frame<T>::propagate, src/Cell/PoolCell_Frame.cpp:123-174, walks them with the rows of the
    // unit map that belong to each; an output pools nothing from the other inputs): the pooling of all inputs' channels, one
    // input behind the other, gathered by one extra launch.
    void addInput(Cell_Frame_HIP* parent);
    using Cell_Frame_HIP::addInput;
    // The connection map over all inputs' channels, {nbOutputs, nbChannels}: what the `mapping` arguments of the reference's
    // addInput() calls add up to (src/Cell/Cell_Frame.cpp:100-132).  Without a call the cell pools one output per channel
    // (the Mapping.ChannelsPerGroup=1 of N2D2's model files).  An output may pool channels of one input only: the
    // reference adds up one pooling per input there, which no model asks for.  A map set after initialize() takes effect
    // at the next propagate(), where it is checked against the cell's channels as they are then.
    void setMapping(const Tensor<bool>& map);
    ~PoolCell_Frame_HIP();
    void initialize();
    void propagate(bool inference = false);
    // src/Cell/PoolCell_Frame.cpp:263-266
    std::pair<double, double> getOutputsRange() const { return mActivation ? mActivation->getOutputRange() : getOutputsRangeParents(); }
    // Graph-level fusion (DeepNet::planFusion): the convolution that feeds this max pooling, and nothing else, computes it
    // in its own launch (n2d2hip_conv_forward_maxpool) when the device library takes the pair; the convolution's own
    // output is then never written.  Returns false, and changes nothing, when it declines.
    bool fuseFirstConv(Cell_Frame_HIP* conv);
    void clearFusion();
    // Can this cell's launch store its output with a border of zeros around every image?  The launch that also computes
    // the first convolution can, and so can the stand-alone 2x2 / 3x3 max pooling of 16-byte channel groups.
    bool writesHalo() const;
    // The pooling as the device library's descriptor
    n2d2hip_pool_desc poolDescriptor() const { return poolDesc(); }

protected:
    void setOutputsDims();

private:
    n2d2hip_pool_desc poolDesc() const;
    void uploadMapping();
    Cell_Frame_HIP* mFusedConv = nullptr;
    Tensor<bool> mMapping;                   // empty: one output per channel
    unsigned char* mMappingDevice = nullptr; // [output][channel] bytes
    static Registrar<PoolCell> mRegistrar;
};

// --------------------------------------------------------------- ElemWiseCell
// include/Cell/ElemWiseCell.hpp:54-63
class ElemWiseCell : public virtual Cell {
public:
    enum Operation { Sum, AbsSum, EuclideanSum, Prod, Max };
    enum CoeffMode { PerLayer, PerInput, PerChannel };
    typedef std::function<std::shared_ptr<ElemWiseCell>(Network&, const DeepNet&, const std::string&, unsigned int, Operation, CoeffMode,
                                                        const std::vector<Float_T>&, const std::vector<Float_T>&,
                                                        const std::shared_ptr<Activation>&)> RegistryCreate_T;
    static RegistryMap_T& registry() { static RegistryMap_T rMap; return rMap; }
    static const char* Type;
    const char* getType() const { return Type; }
    Operation getOperation() const { return mOperation; }
    const std::vector<Float_T>& getWeights() const { return mWeights; }
    const std::vector<Float_T>& getShifts() const { return mShifts; }

protected:
    ElemWiseCell(Operation operation, CoeffMode mode, const std::vector<Float_T>& weights, const std::vector<Float_T>& shifts)
        : mOperation(operation), mCoeffMode(mode), mWeights(weights), mShifts(shifts) {}
    // src/Cell/ElemWiseCell.cpp:59-88
    std::pair<double, double> elemWiseOutputsRange() const;
    Operation mOperation;
    CoeffMode mCoeffMode;
    std::vector<Float_T> mWeights, mShifts;
};

class ElemWiseCell_Frame_HIP : public ElemWiseCell, public Cell_Frame_HIP {
public:
    ElemWiseCell_Frame_HIP(const DeepNet& deepNet, const std::string& name, unsigned int nbOutputs, Operation operation, CoeffMode mode,
                           const std::vector<Float_T>& weights, const std::vector<Float_T>& shifts,
                           const std::shared_ptr<Activation>& activation);
    ~ElemWiseCell_Frame_HIP();
    static std::shared_ptr<ElemWiseCell> create(Network& /*net*/, const DeepNet& deepNet, const std::string& name, unsigned int nbOutputs,
                                                Operation operation, CoeffMode mode, const std::vector<Float_T>& weights,
                                                const std::vector<Float_T>& shifts, const std::shared_ptr<Activation>& activation)
    {
        return std::make_shared<ElemWiseCell_Frame_HIP>(deepNet, name, nbOutputs, operation, mode, weights, shifts, activation);
    }
    void initialize();
    void propagate(bool inference = false);
    bool prepare();
    void launch();
    // Graph-level fusion (both return false, and change nothing, when the device library declines):
    // the ScalingCell behind input k is applied on the fly and never launched ...
    bool foldInputScaling(size_t k, Cell_Frame_HIP* scaling);
    // ... and the convolution behind input k computes this sum in its epilogue: launch() then runs that one kernel.
    bool fuseIntoConv(size_t k, Cell_Frame_HIP* conv);
    void clearFusion();
    Cell_Frame_HIP* fusedConv() const { return mFusedConv; }
    size_t fusedIndex() const { return mFusedIndex; }
    // ... and a whole residual block in one launch (n2d2hip_bottleneck_*): `reduce` (1x1) -> `conv3x3` -> `expand` (1x1), the
    // convolution that has taken this sum, with `projection` (1x1) on the shortcut; all four read nothing but each other
    // and the block's input, the output of `input`, which must then carry a border of one pixel.
    bool fuseBottleneck(Cell_Frame_HIP* reduce, Cell_Frame_HIP* conv3x3, Cell_Frame_HIP* projection, Cell_Frame_HIP* input);
    Cell_Frame_HIP* bottleneckInput() const { return mBottleneck ? mBottleneckIn : nullptr; }
    // ... or the 3x3 convolution in front of the convolution that has taken this sum, the only reader of its output, in
    // that same launch (n2d2hip_conv_chain_*); its input must carry its padding as a border.
    bool fuseChain(Cell_Frame_HIP* conv3x3);
    Cell_Frame_HIP* chainedConv() const { return mChainConv; }
    bool hasFoldedScaling(size_t k) const { return k < mFoldedScaling.size() && mFoldedScaling[k] != nullptr; }
    // src/Cell/ElemWiseCell_Frame.cpp:313-316
    std::pair<double, double> getOutputsRange() const { return mActivation ? mActivation->getOutputRange() : elemWiseOutputsRange(); }

protected:
    void setOutputsDims();

private:
    n2d2hip_elemwise_t mEw;
    unsigned long mEwActGen;
    std::vector<Cell_Frame_HIP*> mFoldedScaling;  // per input, null = not folded
    Cell_Frame_HIP* mFusedConv;
    size_t mFusedIndex;
    n2d2hip_bottleneck_t mBottleneck = nullptr;
    Cell_Frame_HIP* mBottleneckIn = nullptr;
    std::vector<Cell_Frame_HIP*> mBottleneckCells;
    Cell_Frame_HIP* mChainConv = nullptr;
    static Registrar<ElemWiseCell> mRegistrar;
};

// ---------------------------------------------------------------- ScalingCell
// include/Cell/ScalingCell.hpp:39-43
class ScalingCell : public virtual Cell {
public:
    typedef std::function<std::shared_ptr<ScalingCell>(const DeepNet&, const std::string&, unsigned int, Scaling)> RegistryCreate_T;
    static RegistryMap_T& registry() { static RegistryMap_T rMap; return rMap; }
    static const char* Type;
    const char* getType() const { return Type; }
    const Scaling& getScaling() const { return mScaling; }
    void setScaling(Scaling scaling) { mScaling = std::move(scaling); ++mScalingRevision; }

protected:
    explicit ScalingCell(Scaling scaling) : mScaling(std::move(scaling)), mScalingRevision(0) {}
    // src/Cell/ScalingCell.cpp:68-104
    std::pair<double, double> scalingOutputsRange() const;
    Scaling mScaling;
    unsigned mScalingRevision;
};

template <class T>
class ScalingCell_Frame_HIP : public ScalingCell, public Cell_Frame_HIP {
public:
    ScalingCell_Frame_HIP(const DeepNet& deepNet, const std::string& name, unsigned int nbOutputs, Scaling scaling);
    ~ScalingCell_Frame_HIP();
    static std::shared_ptr<ScalingCell> create(const DeepNet& deepNet, const std::string& name, unsigned int nbOutputs, Scaling scaling)
    {
        return std::make_shared<ScalingCell_Frame_HIP<T> >(deepNet, name, nbOutputs, std::move(scaling));
    }
    void initialize();
    void propagate(bool inference = false);
    bool prepare();
    void launch();
    n2d2hip_act_t scalingHandle() const { return mScalingAct; }
    // src/Cell/ScalingCell_Frame.cpp:93-96
    std::pair<double, double> getOutputsRange() const { return mActivation ? mActivation->getOutputRange() : scalingOutputsRange(); }

protected:
    void setOutputsDims();

private:
    n2d2hip_act_t mScalingAct;
    unsigned mBuiltRevision;
    int mBuiltUnsigned;
    static Registrar<ScalingCell> mRegistrar;
};

// ------------------------------------------------------------------ quantizers
// Solver used by the quantizers' update() (include/Solver/SGDSolver_Frame.hpp:84-109: N2D2 ADDS
// rate/(batch*iterationSize)*diff, because its diffInputs carry target - output).
class SGDSolver {
public:
    typedef std::function<std::shared_ptr<SGDSolver>()> RegistryCreate_T;
    static RegistryMap_T& registry() { static RegistryMap_T rMap; return rMap; }
    SGDSolver() : mLearningRate(0.01), mMomentum(0.0), mDecay(0.0), mIterationSize(1), mIterationPass(0), mNbIterations(0),
                  mMomentumData(nullptr), mMomentumSize(0) {}
    virtual ~SGDSolver();
    SGDSolver(const SGDSolver&) = delete;
    SGDSolver& operator=(const SGDSolver&) = delete;
    // LearningRate (0.01), Momentum (0.0), Decay (0.0), IterationSize (1): src/Solver/SGDSolver.cpp:26-41
    void setParameter(const std::string& name, double value);
    bool isNewIteration() const { return mIterationPass == 0; }
    // SGDSolver::getLearningRate with LearningRatePolicy None (src/Solver/SGDSolver.cpp:99-189): 0 on every pass of an
    // iteration but the last
    double getLearningRate();
    unsigned int nbIterations() const { return mNbIterations; }
    // scalar parameter update on the host
    void update(float& data, float diff, unsigned int batchSize);
    // update of n device floats (include/Solver/SGDSolver_Frame.hpp:77-146); one solver serves one tensor, as in the
    // reference, because it owns that tensor's momentum
    void update(float* data, const float* diff, std::size_t n, unsigned int batchSize, void* stream = nullptr);

protected:
    double mLearningRate, mMomentum, mDecay;
    unsigned int mIterationSize, mIterationPass, mNbIterations;
    float* mMomentumData;
    std::size_t mMomentumSize;
};
template <class T>
class SGDSolver_Frame_HIP : public SGDSolver {
public:
    static std::shared_ptr<SGDSolver> create() { return std::make_shared<SGDSolver_Frame_HIP<T> >(); }
private:
    static Registrar<SGDSolver> mRegistrar;
};

// include/Quantizer/QAT/Cell/QuantizerCell.hpp:25-66: Range (255), QuantMode
class QuantizerCell {
public:
    enum QuantMode { Default, Symmetric, Asymmetric, FullRange };
    virtual ~QuantizerCell() {}
    void setRange(std::size_t range) { mRange = range; }
    void setQuantMode(QuantMode mode) { mQuantMode = mode; }
    std::size_t getRange() const { return mRange; }
    QuantMode getQuantMode() const { return mQuantMode; }
    virtual const char* getType() const = 0;
    void setSolver(const std::shared_ptr<SGDSolver>& solver) { mSolver = solver; }
    // device float buffers of n weights: full precision, and the gradient w.r.t. the quantized weights
    virtual void addWeights(float* weights, float* diffQuantizedWeights, std::size_t size, std::size_t outputsSize) = 0;
    virtual void initialize() = 0;
    virtual void propagate() = 0;
    virtual void back_propagate() = 0;
    virtual void update(unsigned int batchSize) = 0;
    virtual float* getQuantizedWeights(unsigned int k) = 0;
    virtual float* getDiffFullPrecisionWeights(unsigned int k) = 0;

protected:
    QuantizerCell() : mRange(255), mQuantMode(Default) {}
    std::size_t mRange;
    QuantMode mQuantMode;
    std::shared_ptr<SGDSolver> mSolver;
};

struct QuantizerBuffers {
    float *fp, *diffQ, *q, *diffFp;
    std::size_t size, outputsSize;
};

// src/Quantizer/QAT/Cell/SAT/SATQuantizerCell.cpp:28-33: ApplyQuantization (true), ApplyScaling (false)
class SATQuantizerCell : public QuantizerCell {
public:
    typedef std::function<std::shared_ptr<SATQuantizerCell>()> RegistryCreate_T;
    static RegistryMap_T& registry() { static RegistryMap_T rMap; return rMap; }
    static const char* Type;
    const char* getType() const { return Type; }
    void setQuantization(bool v) { mApplyQuantization = v; }
    void setScaling(bool v) { mApplyScaling = v; }
    bool getScaling() const { return mApplyScaling; }
protected:
    SATQuantizerCell() : mApplyQuantization(true), mApplyScaling(false) {}
    bool mApplyQuantization, mApplyScaling;
};

// src/Quantizer/QAT/Cell/SAT/SATQuantizerCell_Frame.cpp:65-294
template <class T>
class SATQuantizerCell_Frame_HIP : public SATQuantizerCell {
public:
    SATQuantizerCell_Frame_HIP() : mOutputsSize(0), mStats(nullptr), mWorkspace(nullptr), mWorkspaceBytes(0), mStream(nullptr) {}
    ~SATQuantizerCell_Frame_HIP();
    static std::shared_ptr<SATQuantizerCell> create() { return std::make_shared<SATQuantizerCell_Frame_HIP<T> >(); }
    void addWeights(float* weights, float* diffQuantizedWeights, std::size_t size, std::size_t outputsSize);
    void initialize();
    void propagate();
    void back_propagate();
    void update(unsigned int /*batchSize*/) {}           // nothing to do for SAT in cell mode
    float* getQuantizedWeights(unsigned int k) { return mW.at(k).q; }
    float* getDiffFullPrecisionWeights(unsigned int k) { return mW.at(k).diffFp; }
    // {tanh_max, scaling} of tensor k, read back from the device
    std::pair<float, float> getStats(unsigned int k) const;
    int satMode() const;

private:
    std::vector<QuantizerBuffers> mW;
    std::size_t mOutputsSize;
    float* mStats;          // 2 floats per tensor
    void* mWorkspace;
    std::size_t mWorkspaceBytes;
    void* mStream;
    static Registrar<SATQuantizerCell> mRegistrar;
};

// include/Quantizer/QAT/Activation/QuantizerActivation.hpp:23-25: Range (255)
class QuantizerActivation {
public:
    virtual ~QuantizerActivation() {}
    void setRange(std::size_t range) { mRange = range; }
    std::size_t getRange() const { return mRange; }
    virtual const char* getType() const = 0;
    void setSolver(const std::shared_ptr<SGDSolver>& solver) { mSolver = solver; }
    // in-place on a device float buffer
    virtual void propagate(float* inOut, std::size_t size, bool inference) = 0;
    virtual void back_propagate(const float* diffInput, float* diffOutput, std::size_t size) = 0;
    virtual void update(unsigned int batchSize) = 0;

protected:
    QuantizerActivation() : mRange(255) {}
    std::size_t mRange;
    std::shared_ptr<SGDSolver> mSolver;
};

// src/Quantizer/QAT/Activation/SAT/SATQuantizerActivation_Frame.cpp:73-143: Alpha (1.0)
class SATQuantizerActivation : public QuantizerActivation {
public:
    typedef std::function<std::shared_ptr<SATQuantizerActivation>()> RegistryCreate_T;
    static RegistryMap_T& registry() { static RegistryMap_T rMap; return rMap; }
    static const char* Type;
    const char* getType() const { return Type; }
    void setAlpha(double alpha) { mAlphaParameter = alpha; }
protected:
    SATQuantizerActivation() : mAlphaParameter(1.0) {}
    double mAlphaParameter;
};

template <class T>
class SATQuantizerActivation_Frame_HIP : public SATQuantizerActivation {
public:
    // default solver as in the reference's constructor (SATQuantizerActivation_Frame.cpp:56-64)
    SATQuantizerActivation_Frame_HIP() : mDev(nullptr), mFp(nullptr), mFpSize(0), mWorkspace(nullptr), mWorkspaceBytes(0), mStream(nullptr)
    {
        mSolver = std::make_shared<SGDSolver_Frame_HIP<T> >();
    }
    ~SATQuantizerActivation_Frame_HIP();
    static std::shared_ptr<SATQuantizerActivation> create() { return std::make_shared<SATQuantizerActivation_Frame_HIP<T> >(); }
    void propagate(float* inOut, std::size_t size, bool inference);
    void back_propagate(const float* diffInput, float* diffOutput, std::size_t size);
    void update(unsigned int batchSize);
    float getAlpha();
    float getDiffAlpha();

private:
    void lazyInit(std::size_t size, bool needCopy);
    float* mDev;            // {alpha, diffAlpha}
    float* mFp;             // full-precision copy saved by the training forward
    std::size_t mFpSize;
    void* mWorkspace;
    std::size_t mWorkspaceBytes;
    void* mStream;
    static Registrar<SATQuantizerActivation> mRegistrar;
};

// src/Quantizer/QAT/Cell/LSQ/LSQQuantizerCell.cpp:28-33: StepSize (100), SetOptInitStepSize (true)
class LSQQuantizerCell : public QuantizerCell {
public:
    typedef std::function<std::shared_ptr<LSQQuantizerCell>()> RegistryCreate_T;
    static RegistryMap_T& registry() { static RegistryMap_T rMap; return rMap; }
    static const char* Type;
    const char* getType() const { return Type; }
    void setStepSizeValue(float v) { mStepSizeVal = v; }
    void setOptInitStepSize(bool v) { mSetOptInitStepSize = v; }
protected:
    LSQQuantizerCell() : mStepSizeVal(100.0f), mSetOptInitStepSize(true) {}
    float mStepSizeVal;
    bool mSetOptInitStepSize;
};

// src/Quantizer/QAT/Cell/LSQ/LSQQuantizerCell_Frame.cpp:106-310
template <class T>
class LSQQuantizerCell_Frame_HIP : public LSQQuantizerCell {
public:
    LSQQuantizerCell_Frame_HIP() : mLo(0), mHi(0), mGradScale(0.0f), mDev(nullptr), mWorkspace(nullptr), mWorkspaceBytes(0), mInitialized(false) {}
    ~LSQQuantizerCell_Frame_HIP();
    static std::shared_ptr<LSQQuantizerCell> create() { return std::make_shared<LSQQuantizerCell_Frame_HIP<T> >(); }
    void addWeights(float* weights, float* diffQuantizedWeights, std::size_t size, std::size_t outputsSize);
    void initialize();
    void propagate();
    void back_propagate();
    void update(unsigned int batchSize);
    float* getQuantizedWeights(unsigned int k) { return mW.at(k).q; }
    float* getDiffFullPrecisionWeights(unsigned int k) { return mW.at(k).diffFp; }
    float getStepSize();
    float getDiffStepSize();
    std::pair<int, int> getBitRanges() const { return std::make_pair(mLo, mHi); }

private:
    std::vector<QuantizerBuffers> mW;
    int mLo, mHi;
    float mGradScale;
    float* mDev;            // {stepSize, diffStepSize}
    void* mWorkspace;
    std::size_t mWorkspaceBytes;
    bool mInitialized;
    static Registrar<LSQQuantizerCell> mRegistrar;
};

// src/Quantizer/QAT/Activation/LSQ/LSQQuantizerActivation.cpp:28-33 and ..._Frame.cpp:92-278
class LSQQuantizerActivation : public QuantizerActivation {
public:
    typedef std::function<std::shared_ptr<LSQQuantizerActivation>()> RegistryCreate_T;
    static RegistryMap_T& registry() { static RegistryMap_T rMap; return rMap; }
    static const char* Type;
    const char* getType() const { return Type; }
    void setStepSizeValue(float v) { mStepSizeParameter = v; }
    void setOptInitStepSize(bool v) { mSetOptInitStepSize = v; }
protected:
    LSQQuantizerActivation() : mStepSizeParameter(100.0f), mSetOptInitStepSize(true) {}
    float mStepSizeParameter;
    bool mSetOptInitStepSize;
};

template <class T>
class LSQQuantizerActivation_Frame_HIP : public LSQQuantizerActivation {
public:
    LSQQuantizerActivation_Frame_HIP() : mGradScale(0.0f), mDev(nullptr), mFp(nullptr), mFpSize(0), mWorkspace(nullptr), mWorkspaceBytes(0) {}
    ~LSQQuantizerActivation_Frame_HIP();
    static std::shared_ptr<LSQQuantizerActivation> create() { return std::make_shared<LSQQuantizerActivation_Frame_HIP<T> >(); }
    void propagate(float* inOut, std::size_t size, bool inference);
    void back_propagate(const float* diffInput, float* diffOutput, std::size_t size);
    void update(unsigned int batchSize);
    float getStepSize();
    float getDiffStepSize();

private:
    float mGradScale;
    float* mDev;            // {stepSize, diffStepSize}
    float* mFp;
    std::size_t mFpSize;
    void* mWorkspace;
    std::size_t mWorkspaceBytes;
    static Registrar<LSQQuantizerActivation> mRegistrar;
};

// -------------------------------------------------------------------- DeepNet
// Layer-ordered container: what DeepNet::addCell / getParentCells / propagate provide to the path
// (src/DeepNet.cpp:2692-2719).
class DeepNet {
public:
    DeepNet() {}
    // parents empty = connected to the environment
    void addCell(const std::shared_ptr<Cell>& cell, const std::vector<std::shared_ptr<Cell> >& parents);
    std::shared_ptr<Cell> getCell(const std::string& name) const;
    const std::vector<std::shared_ptr<Cell> >& getCells() const { return mOrder; }
    // environment: integer-valued stimuli {W,H,C,B}
    void setStimuli(unsigned int nbChannels, unsigned int height, unsigned int width, unsigned int batchSize);
    void setStimuliData(const Tensor<Float_T>& data);
    HipTensor& getStimuli() { return mStimuli; }
    void initialize();
    void propagate(bool inference = true);
    void synchronize();
    // Fusion across cells (on by default): a ScalingCell read only by an ElemWise sum is applied inside that sum, and a
    // two-input sum is computed in the epilogue of the 1x1 convolution that produces its later input.  Results are
    // those of the separate cells, bit for bit; the folded cells' own outputs are not written (getOutputs() on them
    // throws).  With it, a tensor written by a convolution and read only by convolutions is stored with the readers'
    // padding as a border of zeros (n2d2hip_tensor::halo).  Turn it off to read every cell's output.
    // What quantization left in the cells beside the free parameters, one text file "<dirName>/<cell>.quant" per cell: the
    // cell's and its activation's bit widths and the activation's (or the ScalingCell's) Scaling.  Together with
    // exportFreeParameters / importFreeParameters this moves a quantized graph between processes.
    void saveQuantization(const std::string& dirName) const;
    void loadQuantization(const std::string& dirName);
    void setFusion(bool enabled);
    bool getFusion() const { return mFusion; }
    // Number of cells propagate() does not launch because a consumer computes them
    size_t nbFoldedCells() const;

private:
    void planFusion();
    void layoutStimuli();
    Tensor<Float_T> mStimuliHost;          // what setStimuliData() was given last
    bool mFusion = true, mPlanned = false;
    std::vector<std::shared_ptr<Cell> > mOrder;
    std::vector<Cell_Frame_HIP*> mFrames;  // mOrder, as the cells' device side
    std::map<std::string, std::shared_ptr<Cell> > mCells;
    HipTensor mStimuli;
    unsigned int mEnvC = 0, mEnvH = 0, mEnvW = 0, mEnvB = 0;
};

// The step of N2D2's post-training quantization that turns the floating-point rescale of a cell into one of the integer
// Scaling modes the quantized cells execute (src/DeepNetQuantization.cpp:1043-1287).  A graph whose activations carry
// FLOAT_MULT scalings (from a calibration done elsewhere) becomes runnable on the integer path this way.
class DeepNetQuantization {
public:
    // Largest number of fractional bits for which every rounded factor fits int16 (FIXED_MULT16, falling back to
    // FIXED_MULT32, which `mode` then says) or int32; at most 50 (src/DeepNetQuantization.cpp:1043-1093)
    static std::pair<std::size_t, std::vector<std::int32_t> > approximateScalingWithFixedPoint(ScalingMode& mode,
                                                                                               const std::vector<Float_T>& scalingPerOutput);
    // scaling <= 1 as a sum of nbDivisions powers of two 2^-e, greedily from the largest; .second is sum / scaling, the
    // factor by which the result overshoots (>= 1; exactly 1 when the greedy sum reaches 98 % of the scaling)
    // (src/DeepNetQuantization.cpp:1095-1134)
    static std::pair<std::vector<unsigned char>, double> approximateScalingWithPowerOf2Divs(Float_T scaling, std::size_t nbDivisions);
    // Replaces the FLOAT_MULT scaling of `activation` by its approximation in `actScalingMode`; for the shift modes the
    // cell's weights and biases are divided by the overshoot, per output (src/DeepNetQuantization.cpp:1147-1178,
    // 1201-1287).  Scalings above 1 cannot be shifts: FIXED_MULT16 is used for that cell instead.
    static void approximateActivationScaling(Cell& cell, Activation& activation, ScalingMode actScalingMode);
};

// include/ScalingMode.hpp:64-67
enum class WeightsApprox { NONE, RINTF };

// What the pass below reads from a trained BatchNormCell (BatchNormCell::getScales / getBiases / getMeans / getVariances,
// its Epsilon) and from the SAT quantizer of that cell's activation (getRange, getAlpha).
struct BatchNormParameters {
    std::vector<double> scales, biases, means, variances;
    double epsilon = 1.0e-5;
    std::size_t actRange = 0;   // 0: the activation has no SAT quantizer (the pass then declines)
    double actAlpha = 0.0;
};

// What it reads from the trained float Conv / Fc cell: the weight quantizer's tensor of the last propagate
// (ConvCell::getQuantWeight; the weights themselves without a quantizer) in the layout the cell holds weights in,
// the biases (empty: NoBias), the quantizer's range (0: none), whether its QuantMode is Default, and the divisor the
// quantizer applied with ApplyScaling (SATQuantizerCell_Frame<T>::getSAT_scaling, 1 otherwise).
struct QATCellParameters {
    Tensor<Float_T> quantWeights, biases;
    std::size_t weightsRange = 0;
    bool defaultQuantMode = true;
    double satScaling = 1.0;
};

// The step that turns a SAT-trained float graph into the integer cells of this library
// (src/Quantizer/QAT/Optimization/DeepNetQAT.cpp).  The reference rewrites each float cell in place; here the trained
// values come in as plain data and the integer cell (model "Frame_HIP") that takes their place is filled: integer
// weights and biases, the number of bits, and an activation Scaling that clips at the activation's alpha and rescales
// accumulator units to the next cell's levels.  The (range, alpha) pairs are threaded through the calls as
// DeepNetQAT::fuseQATGraph does: .first describes the cell's input levels and is replaced by the output's on return.
class DeepNetQAT {
public:
    // Conv followed by BatchNorm (:902-1326).  The cell's activation becomes a Rectifier carrying the Scaling.
    static bool QuantizeAndfuseBatchNormWithConv(std::pair<std::size_t, std::size_t>& rangeConvBN, std::pair<double, double>& alphasConvBN,
                                                 ConvCell& convCell, const QATCellParameters& trained, const BatchNormParameters& bn,
                                                 ScalingMode actScalingMode, WeightsApprox wMode = WeightsApprox::NONE,
                                                 WeightsApprox bMode = WeightsApprox::NONE, WeightsApprox cMode = WeightsApprox::NONE);
    // Fc (:655-900).  actRange 0: the cell's activation has no quantizer.  The activation is kept and receives a
    // FLOAT_MULT Scaling.
    static bool QuantizeFC(std::pair<std::size_t, std::size_t>& rangeOpFc, std::pair<double, double>& alphaOpFC, FcCell& fcCell,
                           const QATCellParameters& trained, std::size_t actRange, double actAlpha,
                           WeightsApprox wMode = WeightsApprox::NONE, WeightsApprox bMode = WeightsApprox::NONE,
                           WeightsApprox cMode = WeightsApprox::NONE);
    // ElemWise (:521-653, as built with CUDA: the CPU-only build of the reference sets the number of bits and nothing
    // else).  The activation becomes a Rectifier with a clipped FLOAT_MULT Scaling.
    static bool QuantizeElemWise(std::pair<std::size_t, std::size_t>& rangeElWise, std::pair<double, double>& alphaElWise,
                                 std::size_t rangeParent0, double alphaParent0, ElemWiseCell& elemWiseCell, std::size_t actRange,
                                 double actAlpha);
};

// Builds a DeepNet from the subset of N2D2's INI format the quantized path needs
// (DefaultModel, [env]/[sp] sizes, Conv / Fc / Pool / ElemWise / Scaling sections with Input=,
// KernelDims / KernelWidth / KernelHeight, NbOutputs, Stride, Padding, Dilation, PoolDims, Pooling, Operation,
// ActivationFunction, Mapping.ChannelsPerGroup=1 for depthwise).  Cells are created through the Registrar
// with the model key found in DefaultModel, as src/Generator/*CellGenerator.cpp do.
std::shared_ptr<DeepNet> generateFromINI(const std::string& iniText, std::string* modelOut = nullptr);

} // namespace N2D2
