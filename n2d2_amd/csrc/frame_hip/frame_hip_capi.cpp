// C entry points over the Frame_HIP host cells, for the Python test-suite and demos: build a net from INI text
// through the Registrar, set parameters the way N2D2's quantization pass leaves them, propagate, read outputs.
// Every function returns 0 on success; the message of the last C++ exception is kept per thread.
#include <cstring>

#include <hip/hip_runtime_api.h>

#include "frame_hip.hpp"

using namespace N2D2;

namespace {
thread_local std::string g_error;
struct Net {
    std::shared_ptr<DeepNet> deepNet;
    std::string model;
};
template <class F>
int guarded(F f)
{
    try {
        f();
        return 0;
    } catch (const std::exception& e) {
        g_error = e.what();
        return 1;
    }
}
Scaling makeScaling(int mode, const void* scaling, size_t n, int fracBits, int isClipped, const float* clip)
{
    std::vector<Float_T> cl;
    if (isClipped && clip) cl.assign(clip, clip + n);
    switch (mode) {
    case N2D2HIP_SCALING_NONE: return Scaling();
    case N2D2HIP_SCALING_FLOAT_MULT:
        return Scaling::floatingPointScaling(std::vector<Float_T>((const float*)scaling, (const float*)scaling + n), isClipped != 0, cl);
    case N2D2HIP_SCALING_FIXED_MULT16:
    case N2D2HIP_SCALING_FIXED_MULT32:
        return Scaling::fixedPointScaling(mode == N2D2HIP_SCALING_FIXED_MULT16 ? ScalingMode::FIXED_MULT16 : ScalingMode::FIXED_MULT32,
                                          (size_t)fracBits, std::vector<std::int32_t>((const std::int32_t*)scaling, (const std::int32_t*)scaling + n),
                                          isClipped != 0, cl);
    case N2D2HIP_SCALING_SINGLE_SHIFT:
        return Scaling::singleShiftScaling(std::vector<unsigned char>((const unsigned char*)scaling, (const unsigned char*)scaling + n), isClipped != 0, cl);
    case N2D2HIP_SCALING_DOUBLE_SHIFT: {
        std::vector<std::pair<unsigned char, unsigned char> > v;
        for (size_t i = 0; i < n; ++i) v.push_back(std::make_pair(((const unsigned char*)scaling)[2 * i], ((const unsigned char*)scaling)[2 * i + 1]));
        return Scaling::doubleShiftScaling(v, isClipped != 0, std::vector<std::pair<unsigned char, unsigned char> >());
    }
    default: throw std::runtime_error("Unsupported scaling propagation.");
    }
}
} // namespace

extern "C" {

const char* fh_last_error(void) { return g_error.c_str(); }

// 1 if a factory is registered for (cell type, model key, float)
int fh_registrar_exists(const char* type, const char* key)
{
    const std::string t(type), k(key);
    if (t == "Conv") return Registrar<ConvCell>::exists<float>(k);
    if (t == "Fc") return Registrar<FcCell>::exists<float>(k);
    if (t == "Pool") return Registrar<PoolCell>::exists<float>(k);
    if (t == "ElemWise") return Registrar<ElemWiseCell>::exists<float>(k);
    if (t == "Scaling") return Registrar<ScalingCell>::exists<float>(k);
    if (t == "Rectifier") return Registrar<RectifierActivation>::exists<float>(k);
    if (t == "Linear") return Registrar<LinearActivation>::exists<float>(k);
    if (t == "SATCell") return Registrar<SATQuantizerCell>::exists<float>(k);
    if (t == "SATAct") return Registrar<SATQuantizerActivation>::exists<float>(k);
    if (t == "LSQCell") return Registrar<LSQQuantizerCell>::exists<float>(k);
    if (t == "LSQAct") return Registrar<LSQQuantizerActivation>::exists<float>(k);
    if (t == "SGDSolver") return Registrar<SGDSolver>::exists<float>(k);
    return -1;
}

// Registers (Conv, "Frame_HIP", float) a second time: returns 1 and leaves the message in fh_last_error()
// when the Registrar throws as the reference's does.
int fh_registrar_duplicate_throws(void)
{
    try {
        Registrar<ConvCell> again("Frame_HIP", ConvCell_Frame_HIP<float>::create, Registrar<ConvCell>::Type<float>());
        return 0;
    } catch (const std::runtime_error& e) {
        g_error = e.what();
        return 1;
    }
}

// 1 when create() on an unknown key yields an empty function (after printing, as the reference does)
int fh_registrar_unknown_key_is_null(const char* key)
{
    return !Registrar<ConvCell>::create<float>(key) ? 1 : 0;
}

void fh_set_globals(int precision, int unsignedData, int envDataUnsigned)
{
    CellExport::mPrecision = precision;
    DeepNetExport::mUnsignedData = unsignedData != 0;
    DeepNetExport::mEnvDataUnsigned = envDataUnsigned != 0;
}

void* fh_net_from_ini(const char* text)
{
    Net* n = new Net();
    const int rc = guarded([&] { n->deepNet = generateFromINI(text, &n->model); });
    if (rc) { delete n; return nullptr; }
    return n;
}
void fh_net_free(void* net) { delete (Net*)net; }
const char* fh_net_model(void* net) { return ((Net*)net)->model.c_str(); }
int fh_net_nb_cells(void* net) { return (int)((Net*)net)->deepNet->getCells().size(); }
int fh_net_set_fusion(void* net, int enabled) { return guarded([&] { ((Net*)net)->deepNet->setFusion(enabled != 0); }); }
int fh_net_nb_folded(void* net) { return (int)((Net*)net)->deepNet->nbFoldedCells(); }
int fh_net_nb_halo(void* net)
{
    int n = 0;
    for (const auto& c : ((Net*)net)->deepNet->getCells())
        n += std::dynamic_pointer_cast<Cell_Frame_HIP>(c)->outputsHalo() > 0 ? 1 : 0;
    return n;
}
int fh_net_initialize(void* net) { return guarded([&] { ((Net*)net)->deepNet->initialize(); }); }
int fh_net_propagate(void* net) { return guarded([&] { ((Net*)net)->deepNet->propagate(true); ((Net*)net)->deepNet->synchronize(); }); }

// data: integer-valued floats in N2D2 order {W,H,C,B} (= NCHW flat)
int fh_net_set_stimuli(void* net, const float* data, int C, int H, int W, int B)
{
    return guarded([&] {
        Tensor<Float_T> t({(size_t)W, (size_t)H, (size_t)C, (size_t)B});
        std::memcpy(t.data(), data, t.size() * sizeof(float));
        ((Net*)net)->deepNet->setStimuliData(t);
    });
}

// dims = {W, H, C, B} of the cell's outputs; unsignedOut = DeepNetExport::isCellOutputUnsigned(cell)
int fh_cell_info(void* net, const char* name, int* dims, int* unsignedOut, char* typeOut, int typeLen)
{
    return guarded([&] {
        auto c = ((Net*)net)->deepNet->getCell(name);
        auto f = std::dynamic_pointer_cast<Cell_Frame_HIP>(c);
        dims[0] = (int)c->getOutputsWidth(); dims[1] = (int)c->getOutputsHeight(); dims[2] = (int)c->getNbOutputs(); dims[3] = (int)f->batchSize();
        *unsignedOut = DeepNetExport::isCellOutputUnsigned(*c) ? 1 : 0;
        if (typeOut && typeLen > 0) { std::strncpy(typeOut, c->getType(), (size_t)typeLen - 1); typeOut[typeLen - 1] = 0; }
    });
}

// Width of the border of zeros that the fusion plan gave the cell's output tensor (0: none), or -1 on error
int fh_cell_outputs_halo(void* net, const char* name)
{
    int halo = -1;
    guarded([&] { halo = std::dynamic_pointer_cast<Cell_Frame_HIP>(((Net*)net)->deepNet->getCell(name))->outputsHalo(); });
    return halo;
}

int fh_cell_set_quantized(void* net, const char* name, int nbBits, int activationNbBits)
{
    return guarded([&] {
        auto c = ((Net*)net)->deepNet->getCell(name);
        c->setQuantized((size_t)nbBits);
        if (c->getActivation() && activationNbBits > 0) c->getActivation()->setQuantized((size_t)activationNbBits);
    });
}

// Conv: weights {kW,kH,C/groups,O} (= OCHW flat); Fc: [O][K]
int fh_cell_set_weights(void* net, const char* name, const float* w, size_t n, int kW, int kH, int Cg, int O, int weightBits)
{
    return guarded([&] {
        auto c = ((Net*)net)->deepNet->getCell(name);
        Tensor<Float_T> t({(size_t)kW, (size_t)kH, (size_t)Cg, (size_t)O});
        if (t.size() != n) throw std::runtime_error("fh_cell_set_weights(): size mismatch");
        std::memcpy(t.data(), w, n * sizeof(float));
        if (auto conv = std::dynamic_pointer_cast<ConvCell>(c)) { conv->setWeights(t); conv->setWeightsPrecision(weightBits); }
        else if (auto fc = std::dynamic_pointer_cast<FcCell>(c)) fc->setWeights(t);
        else throw std::runtime_error("fh_cell_set_weights(): cell has no weights");
    });
}

// map[o + nbOutputs * c] != 0: output o sees channel c
int fh_get_nb_groups(const unsigned char* map, size_t nbOutputs, size_t nbChannels, long* groups, int* regular)
{
    return guarded([&] {
        Tensor<bool> m({nbOutputs, nbChannels}, false);
        for (size_t c = 0; c < nbChannels; ++c)
            for (size_t o = 0; o < nbOutputs; ++o)
                m.set(o, c, map[o + nbOutputs * c] != 0);
        bool isRegular = true;
        *groups = (long)Cell::getNbGroups(m, &isRegular);
        if (regular) *regular = isRegular ? 1 : 0;
    });
}

int fh_cell_set_mapping(void* net, const char* name, const unsigned char* map, size_t nbOutputs, size_t nbChannels)
{
    return guarded([&] {
        auto cell = ((Net*)net)->deepNet->getCell(name);
        auto conv = std::dynamic_pointer_cast<ConvCell>(cell);
        auto pool = std::dynamic_pointer_cast<PoolCell_Frame_HIP<float> >(cell);
        if (!conv && !pool) throw std::runtime_error("fh_cell_set_mapping(): " + std::string(name) + " is neither a Conv nor a Pool");
        Tensor<bool> m({nbOutputs, nbChannels}, false);
        for (size_t c = 0; c < nbChannels; ++c)
            for (size_t o = 0; o < nbOutputs; ++o)
                m.set(o, c, map[o + nbOutputs * c] != 0);
        if (conv) conv->setMapping(m); else pool->setMapping(m);
    });
}

int fh_net_save_quantization(void* net, const char* dirName) { return guarded([&] { ((Net*)net)->deepNet->saveQuantization(dirName); }); }
int fh_net_load_quantization(void* net, const char* dirName) { return guarded([&] { ((Net*)net)->deepNet->loadQuantization(dirName); }); }

int fh_cell_set_biases(void* net, const char* name, const float* b, size_t n)
{
    return guarded([&] {
        auto c = ((Net*)net)->deepNet->getCell(name);
        Tensor<Float_T> t({n});
        std::memcpy(t.data(), b, n * sizeof(float));
        if (auto conv = std::dynamic_pointer_cast<ConvCell>(c)) conv->setBiases(t);
        else if (auto fc = std::dynamic_pointer_cast<FcCell>(c)) fc->setBiases(t);
        else throw std::runtime_error("fh_cell_set_biases(): cell has no biases");
    });
}

// Installs a Scaling in the cell's activation (what fuseScalingCells does), or in a ScalingCell.
int fh_cell_set_scaling(void* net, const char* name, int mode, const void* scaling, size_t n, int fracBits, int isClipped, const float* clip)
{
    return guarded([&] {
        auto c = ((Net*)net)->deepNet->getCell(name);
        Scaling s = makeScaling(mode, scaling, n, fracBits, isClipped, clip);
        if (auto sc = std::dynamic_pointer_cast<ScalingCell>(c)) sc->setScaling(s);
        else if (c->getActivation()) c->getActivation()->setActivationScaling(s);
        else throw std::runtime_error("fh_cell_set_scaling(): cell " + std::string(name) + " has no activation");
    });
}

// Clipping of the cell's activation Scaling: *isClipped, and the per-output values when out has room for them
int fh_cell_get_clipping(void* net, const char* name, int* isClipped, float* out, size_t capacity, size_t* n)
{
    return guarded([&] {
        auto c = ((Net*)net)->deepNet->getCell(name);
        if (!c->getActivation()) throw std::runtime_error("fh_cell_get_clipping(): cell has no activation");
        const Scaling& s = c->getActivation()->getActivationScaling();
        *isClipped = s.getIsClipped() ? 1 : 0;
        *n = s.getClippingPerOutput().size();
        if (out && capacity >= *n) std::copy(s.getClippingPerOutput().begin(), s.getClippingPerOutput().end(), out);
    });
}

// Bits of the cell (weights) and of its activation, and the activation's type name
int fh_cell_get_quantized(void* net, const char* name, int* cellBits, int* activationBits, char* typeOut, int typeLen)
{
    return guarded([&] {
        auto c = ((Net*)net)->deepNet->getCell(name);
        *cellBits = (int)c->getQuantizedNbBits();
        *activationBits = c->getActivation() ? (int)c->getActivation()->getQuantizedNbBits() : 0;
        if (typeOut && typeLen > 0) {
            std::strncpy(typeOut, c->getActivation() ? c->getActivation()->getType() : "", (size_t)typeLen - 1);
            typeOut[typeLen - 1] = 0;
        }
    });
}

// ---- SAT-trained float values into the integer cells (qat_fuse.cpp).  ranges / alphas: the two-element (input, output)
// pairs DeepNetQAT threads through the graph, updated in place.  Rounding modes: 0 NONE, 1 RINTF.
namespace {
QATCellParameters trainedOf(const float* quantWeights, std::vector<size_t> dims, const float* biases, size_t nbOutputs, size_t weightsRange,
                            int defaultMode, double satScaling)
{
    QATCellParameters t;
    t.quantWeights.resize(dims);
    std::memcpy(t.quantWeights.data(), quantWeights, t.quantWeights.size() * sizeof(float));
    if (biases) {
        t.biases.resize({nbOutputs});
        std::memcpy(t.biases.data(), biases, nbOutputs * sizeof(float));
    }
    t.weightsRange = weightsRange;
    t.defaultQuantMode = defaultMode != 0;
    t.satScaling = satScaling;
    return t;
}
ScalingMode scalingModeOf(int mode)
{
    switch (mode) {
    case N2D2HIP_SCALING_FLOAT_MULT: return ScalingMode::FLOAT_MULT;
    case N2D2HIP_SCALING_FIXED_MULT16: return ScalingMode::FIXED_MULT16;
    case N2D2HIP_SCALING_FIXED_MULT32: return ScalingMode::FIXED_MULT32;
    case N2D2HIP_SCALING_SINGLE_SHIFT: return ScalingMode::SINGLE_SHIFT;
    case N2D2HIP_SCALING_DOUBLE_SHIFT: return ScalingMode::DOUBLE_SHIFT;
    default: return ScalingMode::NONE;
    }
}
WeightsApprox approxOf(int m) { return m ? WeightsApprox::RINTF : WeightsApprox::NONE; }
}

int fh_qat_fuse_batchnorm_with_conv(void* net, const char* name, size_t* ranges, double* alphas, const float* quantWeights, int kW, int kH,
                                    int Cg, int O, const float* biases, size_t weightsRange, int defaultMode, const double* bnScales,
                                    const double* bnBiases, const double* bnMeans, const double* bnVariances, double epsilon, size_t actRange,
                                    double actAlpha, int actScalingMode, int wMode, int bMode, int cMode, int* fused)
{
    return guarded([&] {
        auto conv = std::dynamic_pointer_cast<ConvCell>(((Net*)net)->deepNet->getCell(name));
        if (!conv) throw std::runtime_error("fh_qat_fuse_batchnorm_with_conv(): " + std::string(name) + " is not a Conv");
        const QATCellParameters t = trainedOf(quantWeights, {(size_t)kW, (size_t)kH, (size_t)Cg, (size_t)O}, biases, (size_t)O, weightsRange,
                                              defaultMode, 1.0);
        BatchNormParameters bn;
        bn.scales.assign(bnScales, bnScales + O);
        bn.biases.assign(bnBiases, bnBiases + O);
        bn.means.assign(bnMeans, bnMeans + O);
        bn.variances.assign(bnVariances, bnVariances + O);
        bn.epsilon = epsilon;
        bn.actRange = actRange;
        bn.actAlpha = actAlpha;
        std::pair<size_t, size_t> r(ranges[0], ranges[1]);
        std::pair<double, double> a(alphas[0], alphas[1]);
        *fused = DeepNetQAT::QuantizeAndfuseBatchNormWithConv(r, a, *conv, t, bn, scalingModeOf(actScalingMode), approxOf(wMode), approxOf(bMode),
                                                              approxOf(cMode)) ? 1 : 0;
        ranges[0] = r.first; ranges[1] = r.second;
        alphas[0] = a.first; alphas[1] = a.second;
    });
}

int fh_qat_quantize_fc(void* net, const char* name, size_t* ranges, double* alphas, const float* quantWeights, int K, int O, const float* biases,
                       size_t weightsRange, double satScaling, size_t actRange, double actAlpha, int wMode, int bMode, int cMode)
{
    return guarded([&] {
        auto fc = std::dynamic_pointer_cast<FcCell>(((Net*)net)->deepNet->getCell(name));
        if (!fc) throw std::runtime_error("fh_qat_quantize_fc(): " + std::string(name) + " is not a Fc");
        const QATCellParameters t = trainedOf(quantWeights, {(size_t)1, (size_t)1, (size_t)K, (size_t)O}, biases, (size_t)O, weightsRange, 1, satScaling);
        std::pair<size_t, size_t> r(ranges[0], ranges[1]);
        std::pair<double, double> a(alphas[0], alphas[1]);
        DeepNetQAT::QuantizeFC(r, a, *fc, t, actRange, actAlpha, approxOf(wMode), approxOf(bMode), approxOf(cMode));
        ranges[0] = r.first; ranges[1] = r.second;
        alphas[0] = a.first; alphas[1] = a.second;
    });
}

int fh_qat_quantize_elemwise(void* net, const char* name, size_t* ranges, double* alphas, size_t rangeParent0, double alphaParent0, size_t actRange,
                             double actAlpha)
{
    return guarded([&] {
        auto ew = std::dynamic_pointer_cast<ElemWiseCell>(((Net*)net)->deepNet->getCell(name));
        if (!ew) throw std::runtime_error("fh_qat_quantize_elemwise(): " + std::string(name) + " is not an ElemWise");
        std::pair<size_t, size_t> r(ranges[0], ranges[1]);
        std::pair<double, double> a(alphas[0], alphas[1]);
        DeepNetQAT::QuantizeElemWise(r, a, rangeParent0, alphaParent0, *ew, actRange, actAlpha);
        ranges[0] = r.first; ranges[1] = r.second;
        alphas[0] = a.first; alphas[1] = a.second;
    });
}

// ---- ingestion of a trained / calibrated network (quantization.cpp)
int fh_cell_import_free_parameters(void* net, const char* name, const char* fileName, int ignoreNotExists)
{
    return guarded([&] { ((Net*)net)->deepNet->getCell(name)->importFreeParameters(fileName, ignoreNotExists != 0); });
}

int fh_cell_export_free_parameters(void* net, const char* name, const char* fileName)
{
    return guarded([&] { ((Net*)net)->deepNet->getCell(name)->exportFreeParameters(fileName); });
}

// what = 0: weights, 1: biases.  Returns the element count through *n; copies when out has room for it.
int fh_cell_get_free_parameters(void* net, const char* name, int what, float* out, size_t capacity, size_t* n)
{
    return guarded([&] {
        auto c = ((Net*)net)->deepNet->getCell(name);
        const Tensor<Float_T>* t = nullptr;
        if (auto conv = std::dynamic_pointer_cast<ConvCell>(c)) t = what == 0 ? &conv->getWeights() : &conv->getBiases();
        else if (auto fc = std::dynamic_pointer_cast<FcCell>(c)) t = what == 0 ? &fc->getWeights() : &fc->getBiases();
        else throw std::runtime_error("fh_cell_get_free_parameters(): cell has no free parameters");
        *n = t->empty() ? 0 : t->size();
        if (out && capacity >= *n && *n > 0) std::memcpy(out, t->data(), *n * sizeof(float));
    });
}

// mode: N2D2HIP_SCALING_FIXED_MULT16 / _FIXED_MULT32; *modeOut is the mode finally used
int fh_approximate_scaling_with_fixed_point(int mode, const float* scaling, size_t n, int* modeOut, int* nbFractionalBits, std::int32_t* out)
{
    return guarded([&] {
        ScalingMode m = mode == N2D2HIP_SCALING_FIXED_MULT16 ? ScalingMode::FIXED_MULT16 : ScalingMode::FIXED_MULT32;
        const auto r = DeepNetQuantization::approximateScalingWithFixedPoint(m, std::vector<Float_T>(scaling, scaling + n));
        *modeOut = m == ScalingMode::FIXED_MULT16 ? N2D2HIP_SCALING_FIXED_MULT16 : N2D2HIP_SCALING_FIXED_MULT32;
        *nbFractionalBits = (int)r.first;
        std::copy(r.second.begin(), r.second.end(), out);
    });
}

int fh_approximate_scaling_with_power_of_2_divs(float scaling, int nbDivisions, unsigned char* exponents, double* precision)
{
    return guarded([&] {
        const auto r = DeepNetQuantization::approximateScalingWithPowerOf2Divs(scaling, (size_t)nbDivisions);
        std::copy(r.first.begin(), r.first.end(), exponents);
        *precision = r.second;
    });
}

// Turns the FLOAT_MULT scaling of the cell's activation into `mode` (N2D2HIP_SCALING_*), rescaling the cell's parameters
// where the approximation overshoots
int fh_cell_approximate_activation_scaling(void* net, const char* name, int mode)
{
    return guarded([&] {
        auto c = ((Net*)net)->deepNet->getCell(name);
        if (!c->getActivation()) throw std::runtime_error("fh_cell_approximate_activation_scaling(): cell has no activation");
        static const ScalingMode modes[] = {ScalingMode::NONE, ScalingMode::FLOAT_MULT, ScalingMode::FIXED_MULT16, ScalingMode::FIXED_MULT32,
                                            ScalingMode::SINGLE_SHIFT, ScalingMode::DOUBLE_SHIFT};
        if (mode < 0 || mode > 5) throw std::runtime_error("Unsupported scaling mode.");
        DeepNetQuantization::approximateActivationScaling(*c, *c->getActivation(), modes[mode]);
    });
}

// The activation's Scaling: *mode (N2D2HIP_SCALING_*), *fracBits, and its per-output values as doubles (float factors,
// fixed-point integers, shifts; two per output for DOUBLE_SHIFT); *n = number of values
int fh_cell_get_scaling(void* net, const char* name, int* mode, int* fracBits, double* out, size_t capacity, size_t* n)
{
    return guarded([&] {
        auto c = ((Net*)net)->deepNet->getCell(name);
        if (!c->getActivation()) throw std::runtime_error("fh_cell_get_scaling(): cell has no activation");
        const Scaling& s = c->getActivation()->getActivationScaling();
        std::vector<double> v;
        switch (s.getMode()) {
        case ScalingMode::NONE: *mode = N2D2HIP_SCALING_NONE; break;
        case ScalingMode::FLOAT_MULT: *mode = N2D2HIP_SCALING_FLOAT_MULT; v.assign(s.getFloatScalingPerOutput().begin(), s.getFloatScalingPerOutput().end()); break;
        case ScalingMode::FIXED_MULT16: *mode = N2D2HIP_SCALING_FIXED_MULT16; v.assign(s.getFixedScalingPerOutput().begin(), s.getFixedScalingPerOutput().end()); break;
        case ScalingMode::FIXED_MULT32: *mode = N2D2HIP_SCALING_FIXED_MULT32; v.assign(s.getFixedScalingPerOutput().begin(), s.getFixedScalingPerOutput().end()); break;
        case ScalingMode::SINGLE_SHIFT: *mode = N2D2HIP_SCALING_SINGLE_SHIFT; v.assign(s.getShiftScalingPerOutput().begin(), s.getShiftScalingPerOutput().end()); break;
        case ScalingMode::DOUBLE_SHIFT: *mode = N2D2HIP_SCALING_DOUBLE_SHIFT; v.assign(s.getShiftScalingPerOutput().begin(), s.getShiftScalingPerOutput().end()); break;
        }
        *fracBits = (int)s.getFractionalBits();
        *n = v.size();
        if (out && capacity >= v.size()) std::copy(v.begin(), v.end(), out);
    });
}

int fh_cell_get_outputs(void* net, const char* name, float* out, size_t n)
{
    return guarded([&] {
        auto f = std::dynamic_pointer_cast<Cell_Frame_HIP>(((Net*)net)->deepNet->getCell(name));
        const Tensor<Float_T>& t = f->getOutputs();
        if (t.size() != n) throw std::runtime_error("fh_cell_get_outputs(): size mismatch");
        std::memcpy(out, t.data(), n * sizeof(float));
    });
}

// The DeepNet behind a net handle, for the hooks of other files that fill its cells
void* fh_net_deepnet(void* net) { return ((Net*)net)->deepNet.get(); }

int fh_cell_get_max_output(void* net, const char* name, unsigned int batchPos, unsigned int* out)
{
    return guarded([&] {
        auto f = std::dynamic_pointer_cast<Cell_Frame_HIP>(((Net*)net)->deepNet->getCell(name));
        *out = f->getMaxOutput(batchPos);
    });
}

// what: 0 backPropagate, 1 update, 2 checkGradient: each throws on the inference cells
int fh_cell_learn_step(void* net, const char* name, int what)
{
    return guarded([&] {
        auto f = std::dynamic_pointer_cast<Cell_Frame_HIP>(((Net*)net)->deepNet->getCell(name));
        if (what == 0) f->backPropagate();
        else if (what == 1) f->update();
        else f->checkGradient(1.0e-3, 1.0e-3);
    });
}

// Rewires `name` from the output of `oldParent` to that of `newParent` (Cell_Frame<T>::replaceInput); oldParent may
// name a cell that is not an input of `name`, which is the error case.
int fh_cell_replace_input(void* net, const char* name, const char* oldParent, const char* newParent)
{
    return guarded([&] {
        auto dn = ((Net*)net)->deepNet;
        auto f = std::dynamic_pointer_cast<Cell_Frame_HIP>(dn->getCell(name));
        auto o = std::dynamic_pointer_cast<Cell_Frame_HIP>(dn->getCell(oldParent));
        auto n = std::dynamic_pointer_cast<Cell_Frame_HIP>(dn->getCell(newParent));
        f->replaceInput(o->getDeviceOutputs(), n->getDeviceOutputs(), n.get());
    });
}

// ---- quantizers, each created through the Registrar under the given model key.  Host buffers in and out.
int fh_sat_cell_run(const char* model, const float* w, const float* diffQ, size_t n, size_t outputsSize, int range, int quantMode,
                    int applyQuantization, int applyScaling, float* wq, float* diffW, float* stats)
{
    return guarded([&] {
        auto f = Registrar<SATQuantizerCell>::create<float>(model);
        if (!f) throw std::runtime_error("Quantizer model \"" + std::string(model) + "\" is not valid");
        auto q = std::dynamic_pointer_cast<SATQuantizerCell_Frame_HIP<float> >(f());
        float *dW = nullptr, *dD = nullptr;
        if (hipMalloc((void**)&dW, n * 4) != hipSuccess || hipMalloc((void**)&dD, n * 4) != hipSuccess) throw std::runtime_error("hipMalloc");
        hipMemcpy(dW, w, n * 4, hipMemcpyHostToDevice);
        hipMemcpy(dD, diffQ, n * 4, hipMemcpyHostToDevice);
        q->setRange((size_t)range);
        q->setQuantMode((QuantizerCell::QuantMode)quantMode);
        q->setQuantization(applyQuantization != 0);
        q->setScaling(applyScaling != 0);
        q->addWeights(dW, dD, n, outputsSize);
        q->initialize();
        q->propagate();
        q->back_propagate();
        hipDeviceSynchronize();
        hipMemcpy(wq, q->getQuantizedWeights(0), n * 4, hipMemcpyDeviceToHost);
        hipMemcpy(diffW, q->getDiffFullPrecisionWeights(0), n * 4, hipMemcpyDeviceToHost);
        const auto st = q->getStats(0);
        stats[0] = st.first; stats[1] = st.second;
        q.reset();
        hipFree(dW); hipFree(dD);
    });
}

// Two training passes inside one solver iteration (IterationSize = 2) then an update: alphas[0..2] = alpha before,
// accumulated diffAlpha, alpha after the solver step.
int fh_sat_act_run(const char* model, const float* x, const float* diffIn, size_t n, int range, float alpha, float learningRate, float* y,
                   float* diffOut, float* alphas)
{
    return guarded([&] {
        auto f = Registrar<SATQuantizerActivation>::create<float>(model);
        auto fs = Registrar<SGDSolver>::create<float>(model);
        if (!f || !fs) throw std::runtime_error("Quantizer model \"" + std::string(model) + "\" is not valid");
        auto q = std::dynamic_pointer_cast<SATQuantizerActivation_Frame_HIP<float> >(f());
        auto solver = fs();
        solver->setParameter("LearningRate", learningRate);
        solver->setParameter("IterationSize", 2);
        q->setSolver(solver);
        q->setRange((size_t)range);
        q->setAlpha(alpha);
        float *dX = nullptr, *dG = nullptr, *dO = nullptr;
        if (hipMalloc((void**)&dX, n * 4) != hipSuccess || hipMalloc((void**)&dG, n * 4) != hipSuccess || hipMalloc((void**)&dO, n * 4) != hipSuccess)
            throw std::runtime_error("hipMalloc");
        hipMemcpy(dG, diffIn, n * 4, hipMemcpyHostToDevice);
        for (int pass = 0; pass < 2; ++pass) {
            hipMemcpy(dX, x, n * 4, hipMemcpyHostToDevice);
            q->propagate(dX, n, false);
            q->back_propagate(dG, dO, n);          // pass 0: new iteration (beta 0); pass 1: accumulates (beta 1)
            if (pass == 0) { alphas[0] = q->getAlpha(); q->update(1); }     // first pass of the iteration: no parameter step yet
        }
        hipDeviceSynchronize();
        alphas[1] = q->getDiffAlpha();
        q->update(1);
        alphas[2] = q->getAlpha();
        hipMemcpy(y, dX, n * 4, hipMemcpyDeviceToHost);
        hipMemcpy(diffOut, dO, n * 4, hipMemcpyDeviceToHost);
        q.reset();
        hipFree(dX); hipFree(dG); hipFree(dO);
    });
}

int fh_lsq_cell_run(const char* model, const float* w, const float* diffQ, size_t n, int range, float stepSize, int optInit, float* wq,
                    float* diffW, float* steps)
{
    return guarded([&] {
        auto f = Registrar<LSQQuantizerCell>::create<float>(model);
        if (!f) throw std::runtime_error("Quantizer model \"" + std::string(model) + "\" is not valid");
        auto q = std::dynamic_pointer_cast<LSQQuantizerCell_Frame_HIP<float> >(f());
        float *dW = nullptr, *dD = nullptr;
        if (hipMalloc((void**)&dW, n * 4) != hipSuccess || hipMalloc((void**)&dD, n * 4) != hipSuccess) throw std::runtime_error("hipMalloc");
        hipMemcpy(dW, w, n * 4, hipMemcpyHostToDevice);
        hipMemcpy(dD, diffQ, n * 4, hipMemcpyHostToDevice);
        q->setRange((size_t)range);
        q->setStepSizeValue(stepSize);
        q->setOptInitStepSize(optInit != 0);
        q->addWeights(dW, dD, n, 1);
        q->initialize();
        q->propagate();
        q->back_propagate();
        hipDeviceSynchronize();
        hipMemcpy(wq, q->getQuantizedWeights(0), n * 4, hipMemcpyDeviceToHost);
        hipMemcpy(diffW, q->getDiffFullPrecisionWeights(0), n * 4, hipMemcpyDeviceToHost);
        steps[0] = q->getStepSize();
        steps[1] = q->getDiffStepSize();
        steps[2] = (float)q->getBitRanges().first;
        steps[3] = (float)q->getBitRanges().second;
        q.reset();
        hipFree(dW); hipFree(dD);
    });
}

int fh_lsq_act_run(const char* model, const float* x, const float* diffIn, size_t n, int range, float stepSize, int optInit, float* y,
                   float* diffOut, float* steps)
{
    return guarded([&] {
        auto f = Registrar<LSQQuantizerActivation>::create<float>(model);
        if (!f) throw std::runtime_error("Quantizer model \"" + std::string(model) + "\" is not valid");
        auto q = std::dynamic_pointer_cast<LSQQuantizerActivation_Frame_HIP<float> >(f());
        q->setRange((size_t)range);
        q->setStepSizeValue(stepSize);
        q->setOptInitStepSize(optInit != 0);
        float *dX = nullptr, *dG = nullptr, *dO = nullptr;
        if (hipMalloc((void**)&dX, n * 4) != hipSuccess || hipMalloc((void**)&dG, n * 4) != hipSuccess || hipMalloc((void**)&dO, n * 4) != hipSuccess)
            throw std::runtime_error("hipMalloc");
        hipMemcpy(dX, x, n * 4, hipMemcpyHostToDevice);
        hipMemcpy(dG, diffIn, n * 4, hipMemcpyHostToDevice);
        q->propagate(dX, n, false);
        q->back_propagate(dG, dO, n);
        hipDeviceSynchronize();
        hipMemcpy(y, dX, n * 4, hipMemcpyDeviceToHost);
        hipMemcpy(diffOut, dO, n * 4, hipMemcpyDeviceToHost);
        steps[0] = q->getStepSize();
        steps[1] = q->getDiffStepSize();
        q.reset();
        hipFree(dX); hipFree(dG); hipFree(dO);
    });
}

} // extern "C"
