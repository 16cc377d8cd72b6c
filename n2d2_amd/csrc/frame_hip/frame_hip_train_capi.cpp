// C entry points over the float training cells, for the Python test-suite: build a sequential net of ActivationCell /
// ConvCell / SoftmaxCell through the Registrar, attach SAT or LSQ quantizers, run learning iterations, read parameters.
// Every function returns 0 on success; fh_train_last_error() holds the message of the last C++ exception.
#include <cstring>

#include <hip/hip_runtime_api.h>

#include "frame_hip_train.hpp"

using namespace N2D2;

namespace {
thread_local std::string g_train_error;
template <class F>
int guardedT(F f)
{
    try {
        f();
        return 0;
    } catch (const std::exception& e) {
        g_train_error = e.what();
        return 1;
    }
}

struct TrainNet {
    std::string model;
    Network net;
    DeepNet deepNet;
    DeviceFloats input, inputDiff, inputDiffPreset, targets;
    std::vector<std::shared_ptr<Cell_FrameTrain_HIP> > cells;
    std::map<std::string, std::shared_ptr<SATQuantizerActivation_Frame_HIP<float> > > satAct;
    std::map<std::string, std::shared_ptr<LSQQuantizerActivation_Frame_HIP<float> > > lsqAct;
    std::map<std::string, std::shared_ptr<LSQQuantizerCell_Frame_HIP<float> > > lsqCell;
    std::vector<std::string> nextInputs;      // the cells the next added cell reads (empty: the cell added last)
    Cell_FrameTrain_HIP* byName(const std::string& name)
    {
        for (auto& c : cells)
            if (c->getName() == name) return c.get();
        throw std::runtime_error("No cell named \"" + name + "\"");
    }
    // the cell the next added cell reads first (null: the environment)
    Cell_FrameTrain_HIP* last() { return !nextInputs.empty() ? byName(nextInputs[0]) : (cells.empty() ? nullptr : cells.back().get()); }
};

// act: -1 none, 0 Linear, 1 Rectifier; actQuant: 0 none, 1 SAT (param = alpha), 2 LSQ (param = step size, <= 0: optimal init)
std::shared_ptr<Activation> makeActivation(TrainNet& n, const std::string& name, int act, int actQuant, int range, float param)
{
    if (act < 0)
        return std::shared_ptr<Activation>();
    std::shared_ptr<Activation> a;
    if (act == 0) {
        auto f = Registrar<LinearActivation>::create<float>("Frame_HIP");
        a = f();
    } else {
        auto f = Registrar<RectifierActivation>::create<float>("Frame_HIP");
        a = f();
    }
    if (actQuant == 1) {
        auto q = std::dynamic_pointer_cast<SATQuantizerActivation_Frame_HIP<float> >(Registrar<SATQuantizerActivation>::create<float>("Frame_HIP")());
        q->setRange((size_t)range);
        q->setAlpha(param);
        a->setQuantizer(q);
        n.satAct[name] = q;
    } else if (actQuant == 2) {
        auto q = std::dynamic_pointer_cast<LSQQuantizerActivation_Frame_HIP<float> >(Registrar<LSQQuantizerActivation>::create<float>("Frame_HIP")());
        q->setRange((size_t)range);
        if (param > 0.0f) { q->setStepSizeValue(param); q->setOptInitStepSize(false); }
        q->setSolver(Registrar<SGDSolver>::create<float>("Frame_HIP")());
        a->setQuantizer(q);
        n.lsqAct[name] = q;
    }
    return a;
}

// Cells are added in an order in which every cell follows the cells it reads (propagate runs them in that order,
// backPropagate and update in the reverse one, as DeepNet::learn does over its layers).
void connect(TrainNet& n, const std::shared_ptr<Cell_FrameTrain_HIP>& cell)
{
    if (!n.nextInputs.empty()) {
        for (const std::string& name : n.nextInputs)
            cell->addInput(n.byName(name));
        n.nextInputs.clear();
    } else if (n.cells.empty())
        cell->addInput(n.input, n.inputDiff);
    else
        cell->addInput(n.cells.back().get());
    cell->initialize();
    n.cells.push_back(cell);
}

Cell_FrameTrain_HIP* find(TrainNet& n, const char* name)
{
    for (auto& c : n.cells)
        if (c->getName() == name) return c.get();
    throw std::runtime_error("No cell named \"" + std::string(name) + "\"");
}
} // namespace

extern "C" {

const char* fh_train_last_error(void) { return g_train_error.c_str(); }

int fh_train_registrar_exists(const char* type, const char* key)
{
    const std::string t(type), k(key);
    if (t == "Conv") return Registrar<ConvCell>::exists<float>(k);
    if (t == "Fc") return Registrar<FcCell>::exists<float>(k);
    if (t == "Activation") return Registrar<ActivationCell>::exists<float>(k);
    if (t == "Softmax") return Registrar<SoftmaxCell>::exists<float>(k);
    if (t == "BatchNorm") return Registrar<BatchNormCell>::exists<float>(k);
    if (t == "Pool") return Registrar<PoolCell>::exists<float>(k);
    if (t == "ElemWise") return Registrar<ElemWiseCell>::exists<float>(k);
    return -1;
}

// The environment: a float tensor [B,C,H,W]; propagateGradient != 0 gives the first cell a tensor to write its
// input gradient to (an ActivationCell computes its quantizer's gradient only then, as in the reference).
int fh_train_net_create(const char* model, const float* input, int B, int C, int H, int W, int propagateGradient, void** out)
{
    return guardedT([&] {
        std::unique_ptr<TrainNet> n(new TrainNet);
        n->model = model;
        const std::vector<size_t> dims = {(size_t)W, (size_t)H, (size_t)C, (size_t)B};
        n->input.resize(dims);
        n->input.fromHost(input, n->input.size());
        if (propagateGradient)
            n->inputDiff.resize(dims);
        *out = n.release();
    });
}

void fh_train_net_destroy(void* net) { delete (TrainNet*)net; }

int fh_train_add_activation_cell(void* net, const char* name, int act, int actQuant, int range, float param)
{
    return guardedT([&] {
        TrainNet& n = *(TrainNet*)net;
        auto f = Registrar<ActivationCell>::create<float>(n.model);
        if (!f) throw std::runtime_error("Cell model \"" + n.model + "\" is not valid in section [" + name + "]");
        const unsigned int nbOutputs = n.cells.empty() ? (unsigned int)n.input.dimZ() : n.last()->getNbOutputs();
        auto cell = std::dynamic_pointer_cast<Cell_FrameTrain_HIP>(f(n.deepNet, name, nbOutputs, makeActivation(n, name, act, actQuant, range, param)));
        connect(n, cell);
    });
}

// weights: HOST float [O, C/groups, kH, kW]; bias HOST float [O] or NULL (NoBias).  weightQuant: 0 none, 1 SAT, 2 LSQ.
int fh_train_add_conv(void* net, const char* name, int nbOutputs, int kW, int kH, int strideX, int strideY, int padX, int padY, int depthwise,
                      const float* weights, const float* bias, int act, int actQuant, int actRange, float actParam,
                      int weightQuant, int weightRange, int applyQuantization, int applyScaling, int quantMode)
{
    return guardedT([&] {
        TrainNet& n = *(TrainNet*)net;
        auto f = Registrar<ConvCell>::create<float>(n.model);
        if (!f) throw std::runtime_error("Cell model \"" + n.model + "\" is not valid in section [" + name + "]");
        auto conv = f(n.net, n.deepNet, name, {(unsigned)kW, (unsigned)kH}, (unsigned)nbOutputs, {1U, 1U}, {(unsigned)strideX, (unsigned)strideY},
                      {padX, padY}, {1U, 1U}, makeActivation(n, name, act, actQuant, actRange, actParam));
        auto cell = std::dynamic_pointer_cast<ConvCell_FrameTrain_HIP<float> >(conv);
        const unsigned int nbChannels = n.cells.empty() ? (unsigned int)n.input.dimZ() : n.last()->getNbOutputs();
        const unsigned int groups = depthwise ? nbChannels : 1;
        conv->setNbGroups(groups);
        conv->setParameter("NoBias", bias == nullptr);
        Tensor<Float_T> w({(size_t)kW, (size_t)kH, (size_t)(nbChannels / groups), (size_t)nbOutputs});
        std::memcpy(w.data(), weights, w.size() * sizeof(float));
        conv->setWeights(w);
        if (bias) {
            Tensor<Float_T> b({(size_t)nbOutputs});
            std::memcpy(b.data(), bias, nbOutputs * sizeof(float));
            conv->setBiases(b);
        }
        if (weightQuant == 1) {
            auto q = Registrar<SATQuantizerCell>::create<float>("Frame_HIP")();
            q->setRange((size_t)weightRange);
            q->setQuantization(applyQuantization != 0);
            q->setScaling(applyScaling != 0);
            q->setQuantMode((QuantizerCell::QuantMode)quantMode);
            cell->setQuantizer(q);
        } else if (weightQuant == 2) {
            auto q = Registrar<LSQQuantizerCell>::create<float>("Frame_HIP")();
            q->setRange((size_t)weightRange);
            q->setSolver(Registrar<SGDSolver>::create<float>("Frame_HIP")());
            cell->setQuantizer(q);
            n.lsqCell[name] = std::dynamic_pointer_cast<LSQQuantizerCell_Frame_HIP<float> >(q);
        }
        connect(n, cell);
    });
}

// weights: HOST float [O, C*H*W] (CHW order); bias HOST float [O] or NULL (NoBias).  weightQuant: 0 none, 1 SAT, 2 LSQ.
int fh_train_add_fc(void* net, const char* name, int nbOutputs, const float* weights, const float* bias, int act, int actQuant, int actRange,
                    float actParam, int weightQuant, int weightRange, int applyScaling)
{
    return guardedT([&] {
        TrainNet& n = *(TrainNet*)net;
        auto f = Registrar<FcCell>::create<float>(n.model);
        if (!f) throw std::runtime_error("Cell model \"" + n.model + "\" is not valid in section [" + name + "]");
        auto fc = f(n.net, n.deepNet, name, (unsigned)nbOutputs, makeActivation(n, name, act, actQuant, actRange, actParam));
        auto cell = std::dynamic_pointer_cast<FcCell_FrameTrain_HIP<float> >(fc);
        const size_t K = n.cells.empty() ? n.input.dimX() * n.input.dimY() * n.input.dimZ()
                                         : n.last()->getOutputs().dimX() * n.last()->getOutputs().dimY() * n.last()->getOutputs().dimZ();
        fc->setParameter("NoBias", bias == nullptr);
        Tensor<Float_T> w({K, (size_t)nbOutputs});
        std::memcpy(w.data(), weights, w.size() * sizeof(float));
        fc->setWeights(w);
        if (bias) {
            Tensor<Float_T> b({(size_t)nbOutputs});
            std::memcpy(b.data(), bias, nbOutputs * sizeof(float));
            fc->setBiases(b);
        }
        if (weightQuant == 1) {
            auto q = Registrar<SATQuantizerCell>::create<float>("Frame_HIP")();
            q->setRange((size_t)weightRange);
            q->setScaling(applyScaling != 0);
            cell->setQuantizer(q);
        } else if (weightQuant == 2) {
            auto q = Registrar<LSQQuantizerCell>::create<float>("Frame_HIP")();
            q->setRange((size_t)weightRange);
            q->setSolver(Registrar<SGDSolver>::create<float>("Frame_HIP")());
            cell->setQuantizer(q);
            n.lsqCell[name] = std::dynamic_pointer_cast<LSQQuantizerCell_Frame_HIP<float> >(q);
        }
        connect(n, cell);
    });
}

// params: HOST float [4][nbOutputs] = scales, biases, means, variances, or NULL for the cell's initial values (1, 0, 0, 0)
int fh_train_add_batchnorm(void* net, const char* name, const float* params, double epsilon, double movingAverageMomentum, int act, int actQuant,
                           int actRange, float actParam)
{
    return guardedT([&] {
        TrainNet& n = *(TrainNet*)net;
        auto f = Registrar<BatchNormCell>::create<float>(n.model);
        if (!f) throw std::runtime_error("Cell model \"" + n.model + "\" is not valid in section [" + name + "]");
        const unsigned int nbOutputs = n.cells.empty() ? (unsigned int)n.input.dimZ() : n.last()->getNbOutputs();
        auto bn = f(n.deepNet, name, nbOutputs, makeActivation(n, name, act, actQuant, actRange, actParam));
        bn->setParameter("Epsilon", epsilon);
        bn->setParameter("MovingAverageMomentum", movingAverageMomentum);
        auto cell = std::dynamic_pointer_cast<BatchNormCell_FrameTrain_HIP<float> >(bn);
        if (params) {
            cell->setScales(std::vector<Float_T>(params, params + nbOutputs));
            cell->setBiases(std::vector<Float_T>(params + nbOutputs, params + 2 * nbOutputs));
            cell->setMeans(std::vector<Float_T>(params + 2 * nbOutputs, params + 3 * nbOutputs));
            cell->setVariances(std::vector<Float_T>(params + 3 * nbOutputs, params + 4 * nbOutputs));
        }
        connect(n, cell);
    });
}

// what: 0 scales, 1 biases, 2 running means, 3 running variances, 4 gradient of the scales, 5 gradient of the biases
int fh_train_get_batchnorm(void* net, const char* cell, int what, float* out, size_t n)
{
    return guardedT([&] {
        auto bn = dynamic_cast<BatchNormCell_FrameTrain_HIP<float>*>(find(*(TrainNet*)net, cell));
        if (!bn) throw std::runtime_error("Not a BatchNorm cell: " + std::string(cell));
        const std::vector<Float_T> v = what == 0 ? bn->getScales() : what == 1 ? bn->getBiases() : what == 2 ? bn->getMeans()
                                       : what == 3 ? bn->getVariances() : what == 4 ? bn->getDiffScales() : bn->getDiffBiases();
        if (v.size() != n) throw std::runtime_error("fh_train_get_batchnorm(): size mismatch");
        std::memcpy(out, v.data(), n * sizeof(float));
    });
}

// Max (pooling 0) or Average (pooling 1) pooling, one output per channel
int fh_train_add_pool(void* net, const char* name, int poolW, int poolH, int strideX, int strideY, int padX, int padY, int pooling)
{
    return guardedT([&] {
        TrainNet& n = *(TrainNet*)net;
        auto f = Registrar<PoolCell>::create<float>(n.model);
        if (!f) throw std::runtime_error("Cell model \"" + n.model + "\" is not valid in section [" + name + "]");
        const unsigned int nbOutputs = n.cells.empty() ? (unsigned int)n.input.dimZ() : n.last()->getNbOutputs();
        auto pool = f(n.net, n.deepNet, name, {(unsigned)poolW, (unsigned)poolH}, nbOutputs, {(unsigned)strideX, (unsigned)strideY},
                      {(unsigned)padX, (unsigned)padY}, pooling ? PoolCell::Average : PoolCell::Max, std::shared_ptr<Activation>());
        connect(n, std::dynamic_pointer_cast<Cell_FrameTrain_HIP>(pool));
    });
}

// The cells (comma-separated names) that the cell added next reads, instead of the cell added last.
int fh_train_set_next_inputs(void* net, const char* names)
{
    return guardedT([&] {
        TrainNet& n = *(TrainNet*)net;
        n.nextInputs.clear();
        std::string all(names ? names : ""), item;
        for (size_t i = 0; i <= all.size(); ++i) {
            if (i == all.size() || all[i] == ',') {
                if (!item.empty()) { n.byName(item); n.nextInputs.push_back(item); }
                item.clear();
            } else
                item += all[i];
        }
    });
}

// ElemWise Sum over the inputs set with fh_train_set_next_inputs; weights / shifts: nbCoeffs values each (0: all 1 / all 0)
int fh_train_add_elemwise(void* net, const char* name, const float* weights, const float* shifts, int nbCoeffs, int act, int actQuant, int actRange,
                          float actParam)
{
    return guardedT([&] {
        TrainNet& n = *(TrainNet*)net;
        auto f = Registrar<ElemWiseCell>::create<float>(n.model);
        if (!f) throw std::runtime_error("Cell model \"" + n.model + "\" is not valid in section [" + name + "]");
        if (n.nextInputs.empty()) throw std::runtime_error("fh_train_add_elemwise(): name the inputs first");
        const std::vector<Float_T> w(weights, weights + (weights ? nbCoeffs : 0)), s(shifts, shifts + (shifts ? nbCoeffs : 0));
        auto cell = std::dynamic_pointer_cast<Cell_FrameTrain_HIP>(f(n.net, n.deepNet, name, n.last()->getNbOutputs(), ElemWiseCell::Sum,
                                                                     ElemWiseCell::PerInput, w, s,
                                                                     makeActivation(n, name, act, actQuant, actRange, actParam)));
        connect(n, cell);
    });
}

int fh_train_add_softmax(void* net, const char* name, int withLoss)
{
    return guardedT([&] {
        TrainNet& n = *(TrainNet*)net;
        auto f = Registrar<SoftmaxCell>::create<float>(n.model);
        if (!f) throw std::runtime_error("Cell model \"" + n.model + "\" is not valid in section [" + name + "]");
        if (n.cells.empty()) throw std::runtime_error("A SoftmaxCell needs a parent cell");
        auto cell = std::dynamic_pointer_cast<Cell_FrameTrain_HIP>(f(n.deepNet, name, n.last()->getNbOutputs(), withLoss != 0, 0U));
        connect(n, cell);
    });
}

// Solver parameters of a convolution's weights ("LearningRate", "Momentum", "Decay", "IterationSize")
int fh_train_set_solver_parameter(void* net, const char* cell, const char* name, double value)
{
    return guardedT([&] {
        Cell_FrameTrain_HIP* c = find(*(TrainNet*)net, cell);
        auto s = Registrar<SGDSolver>::create<float>("Frame_HIP")();
        s->setParameter(name, value);
        if (auto conv = dynamic_cast<WeightedCell_FrameTrain_HIP*>(c)) {
            conv->setWeightsSolver(s);
        } else if (auto bn = dynamic_cast<BatchNormCell_FrameTrain_HIP<float>*>(c)) {
            // the scales' and the biases' solvers, one object each
            bn->setScaleSolver(s);
            auto s2 = Registrar<SGDSolver>::create<float>("Frame_HIP")();
            s2->setParameter(name, value);
            bn->setBiasSolver(s2);
        } else {
            throw std::runtime_error("Not a cell with a solver: " + std::string(cell));
        }
    });
}

// targets: HOST float, the shape of the last cell's outputs.  Runs `iterations` times what the reference's learning
// loop runs: propagate front to back, targets into the last cell's diffInputs, applyLoss, backPropagate back to front,
// update back to front.  loss receives the last iteration's.
int fh_train_learn(void* net, const float* targets, size_t nTargets, int iterations, double* loss)
{
    return guardedT([&] {
        TrainNet& n = *(TrainNet*)net;
        if (n.cells.empty()) throw std::runtime_error("Empty net");
        Cell_FrameTrain_HIP* last = n.last();
        if (nTargets != last->getOutputs().size()) throw std::runtime_error("fh_train_learn(): wrong number of targets");
        n.targets.resize(last->getOutputs().dims());
        n.targets.fromHost(targets, nTargets);
        double l = 0.0;
        for (int it = 0; it < iterations; ++it) {
            // the gradient towards the net's input is this iteration's: empty, or what another consumer of the input has
            // already put there (fh_train_preset_input_gradient)
            if (!n.inputDiff.empty()) {
                if (n.inputDiffPreset.empty()) {
                    n.inputDiff.clearValid();
                } else {
                    // (on the stream of the cell that will add to it, like every copy below)
                    if (hipMemcpyAsync(n.inputDiff.data(), n.inputDiffPreset.data(), n.inputDiff.size() * sizeof(float), hipMemcpyDeviceToDevice,
                                       (hipStream_t)n.cells.front()->stream())
                        != hipSuccess)
                        throw std::runtime_error("fh_train_learn(): copy of the preset input gradient failed");
                    n.inputDiff.setValid();
                }
            }
            for (auto& c : n.cells) c->propagate(false);
            if (hipMemcpyAsync(last->getDiffInputs().data(), n.targets.data(), nTargets * sizeof(float), hipMemcpyDeviceToDevice,
                               (hipStream_t)last->stream()) != hipSuccess)
                throw std::runtime_error("fh_train_learn(): copy of the targets failed");
            l = last->applyLoss();
            for (auto c = n.cells.rbegin(); c != n.cells.rend(); ++c) (*c)->backPropagate();
            for (auto c = n.cells.rbegin(); c != n.cells.rend(); ++c) (*c)->update();
        }
        if (hipDeviceSynchronize() != hipSuccess) throw std::runtime_error("fh_train_learn(): device error");
        if (loss) *loss = l;
    });
}

// The chain case of DeepNetQAT::fuseQATGraph (src/Quantizer/QAT/Optimization/DeepNetQAT.cpp:87-520): walks the learning
// cells front to back with the (range, alpha) pairs starting at (255, 255) / (1, 1); every Conv followed by a BatchNorm is
// fused into the integer Conv cell of the same name in `deepNet`, every Fc quantized into the integer Fc of the same name;
// pooling, activation and softmax cells leave the pairs alone.  The learning cells must have propagated once (their
// quantizers hold the quantized weights then).  nbFused receives the number of integer cells filled.
int fh_train_fuse_into(void* net, void* deepNet, int actScalingMode, int wMode, int bMode, int cMode, int* nbFused)
{
    return guardedT([&] {
        TrainNet& n = *(TrainNet*)net;
        DeepNet& target = *(DeepNet*)deepNet;
        const ScalingMode mode = actScalingMode == N2D2HIP_SCALING_FLOAT_MULT ? ScalingMode::FLOAT_MULT
                                 : actScalingMode == N2D2HIP_SCALING_FIXED_MULT16 ? ScalingMode::FIXED_MULT16
                                 : actScalingMode == N2D2HIP_SCALING_FIXED_MULT32 ? ScalingMode::FIXED_MULT32
                                 : actScalingMode == N2D2HIP_SCALING_SINGLE_SHIFT ? ScalingMode::SINGLE_SHIFT : ScalingMode::NONE;
        const WeightsApprox w = wMode ? WeightsApprox::RINTF : WeightsApprox::NONE, b = bMode ? WeightsApprox::RINTF : WeightsApprox::NONE,
                            c = cMode ? WeightsApprox::RINTF : WeightsApprox::NONE;
        std::pair<std::size_t, std::size_t> ranges(255, 255);
        std::pair<double, double> alphas(1.0, 1.0);
        int count = 0;
        for (std::size_t i = 0; i < n.cells.size(); ++i) {
            Cell_FrameTrain_HIP* cell = n.cells[i].get();
            if (auto conv = dynamic_cast<ConvCell_FrameTrain_HIP<float>*>(cell)) {
                auto bn = i + 1 < n.cells.size() ? dynamic_cast<BatchNormCell_FrameTrain_HIP<float>*>(n.cells[i + 1].get()) : nullptr;
                if (!bn)
                    throw std::runtime_error("fh_train_fuse_into(): Conv \"" + conv->getName() + "\" is not followed by a BatchNorm");
                auto dst = std::dynamic_pointer_cast<ConvCell>(target.getCell(conv->getName()));
                if (!dst)
                    throw std::runtime_error("fh_train_fuse_into(): no integer Conv named \"" + conv->getName() + "\"");
                if (i == 0)
                    ranges.first = 255;         // the stimuli: 8 bits
                if (!DeepNetQAT::QuantizeAndfuseBatchNormWithConv(ranges, alphas, *dst, conv->getQATCellParameters(), bn->getBatchNormParameters(),
                                                                  mode, w, b, c))
                    throw std::runtime_error("fh_train_fuse_into(): \"" + bn->getName() + "\" cannot be fused with \"" + conv->getName() + "\"");
                ++count;
                ++i;
            } else if (auto fc = dynamic_cast<FcCell_FrameTrain_HIP<float>*>(cell)) {
                auto dst = std::dynamic_pointer_cast<FcCell>(target.getCell(fc->getName()));
                if (!dst)
                    throw std::runtime_error("fh_train_fuse_into(): no integer Fc named \"" + fc->getName() + "\"");
                std::size_t actRange = 0;
                double actAlpha = 0.0;
                if (fc->getActivation() && fc->getActivation()->getQuantizer()) {
                    auto sat = std::dynamic_pointer_cast<SATQuantizerActivation_Frame_HIP<float> >(fc->getActivation()->getQuantizer());
                    if (!sat)
                        throw std::runtime_error("fh_train_fuse_into(): only SAT activation quantizers can be fused (\"" + fc->getName() + "\")");
                    actRange = sat->getRange();
                    actAlpha = sat->getAlpha();
                }
                DeepNetQAT::QuantizeFC(ranges, alphas, *dst, fc->getQATCellParameters(), actRange, actAlpha, w, b, c);
                ++count;
            }
        }
        if (nbFused) *nbFused = count;
    });
}

// One forward pass; inference != 0 runs the quantizers without saving what backPropagate needs
int fh_train_propagate(void* net, int inference)
{
    return guardedT([&] {
        for (auto& c : ((TrainNet*)net)->cells) c->propagate(inference != 0);
        if (hipDeviceSynchronize() != hipSuccess) throw std::runtime_error("fh_train_propagate(): device error");
    });
}

// what: 0 outputs, 1 diffInputs, 2 weights, 3 gradient of the (quantized) weights, 4 quantized weights
int fh_train_get(void* net, const char* cell, int what, float* out, size_t n)
{
    return guardedT([&] {
        Cell_FrameTrain_HIP* c = find(*(TrainNet*)net, cell);
        Tensor<Float_T> t;
        auto conv = dynamic_cast<WeightedCell_FrameTrain_HIP*>(c);
        if (what == 0) t = c->getOutputs().toHost();
        else if (what == 1) t = c->getDiffInputs().toHost();
        else if (!conv) throw std::runtime_error("Not a cell with weights: " + std::string(cell));
        else if (what == 2) {
            conv->synchronizeWeightsToHost();
            if (auto cc = dynamic_cast<ConvCell*>(c)) t = cc->getWeights();
            else t = dynamic_cast<FcCell*>(c)->getWeights();
        }
        else if (what == 3) t = conv->getDiffWeights();
        else t = conv->getQuantizedWeights();
        if (t.size() != n) throw std::runtime_error("fh_train_get(): size mismatch");
        std::memcpy(out, t.data(), n * sizeof(float));
    });
}

// A gradient towards the net's input that is already there when backPropagate() reaches the first cell, as if another
// consumer of the input had run first: the first cell must add its own to it.
int fh_train_preset_input_gradient(void* net, const float* values, size_t n)
{
    return guardedT([&] {
        TrainNet& t = *(TrainNet*)net;
        if (t.inputDiff.empty() || t.inputDiff.size() != n) throw std::runtime_error("fh_train_preset_input_gradient(): size mismatch");
        t.inputDiffPreset.resize(t.inputDiff.dims());
        t.inputDiffPreset.fromHost(values, n);
    });
}

int fh_train_input_gradient(void* net, float* out, size_t n)
{
    return guardedT([&] {
        const Tensor<Float_T> t = ((TrainNet*)net)->inputDiff.toHost();
        if (t.size() != n) throw std::runtime_error("fh_train_input_gradient(): size mismatch");
        std::memcpy(out, t.data(), n * sizeof(float));
    });
}

// The learned parameter of a cell's activation quantizer: SAT alpha or LSQ step size; grad receives its last gradient
int fh_train_get_activation_quantizer(void* net, const char* cell, float* value, float* grad)
{
    return guardedT([&] {
        TrainNet& n = *(TrainNet*)net;
        auto s = n.satAct.find(cell);
        auto l = n.lsqAct.find(cell);
        if (s != n.satAct.end()) { *value = s->second->getAlpha(); if (grad) *grad = s->second->getDiffAlpha(); }
        else if (l != n.lsqAct.end()) { *value = l->second->getStepSize(); if (grad) *grad = l->second->getDiffStepSize(); }
        else throw std::runtime_error("No activation quantizer on cell \"" + std::string(cell) + "\"");
    });
}

// The learned step size of a cell's LSQ weight quantizer; grad receives its last gradient
int fh_train_get_weight_quantizer(void* net, const char* cell, float* value, float* grad)
{
    return guardedT([&] {
        TrainNet& n = *(TrainNet*)net;
        auto l = n.lsqCell.find(cell);
        if (l == n.lsqCell.end()) throw std::runtime_error("No LSQ weight quantizer on cell \"" + std::string(cell) + "\"");
        *value = l->second->getStepSize();
        if (grad) *grad = l->second->getDiffStepSize();
    });
}

} // extern "C"
