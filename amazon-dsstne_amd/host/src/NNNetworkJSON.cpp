// NNNetworkJSON.cpp — network definition files in JSON (reference: LoadNeuralNetworkJSON, engine/NNNetwork.cpp:2792-3760).
// The file is turned into the same NNNetworkDescriptor the binary loader fills; keys and enumerated values are matched
// without regard to case, unknown keys are errors, "N": "auto" takes a layer's dimensions from the data set of that name,
// layers without "Source" follow the layer before them, and one weight descriptor is made per source.  Fully connected
// layers only are built by this library; convolutional and pooling entries are parsed into the descriptor and refused when
// the network is constructed.  A definition carries no weight values: they are initialised by NNWeight::Randomize.
#include <cmath>
#include <functional>
#include <set>
#include <stdexcept>

#include "Json.h"
#include "amazon/dsstne/engine/NNTypes.h"

namespace {

using json::Value;
using Setter = std::function<void(const Value&)>;
using KeyTable = std::vector<std::pair<const char*, Setter>>;

struct DefinitionError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// Runs the setter registered for a key (lower case); false when the table does not know the key.
bool dispatch(const KeyTable& table, const std::string& key, const Value& v)
{
    for (auto& e : table) {
        if (key == e.first) {
            e.second(v);
            return true;
        }
    }
    return false;
}

// A block of named numeric parameters such as "SparsenessPenalty": {"p": .., "beta": ..}.
void readBlock(const Value& block, const char* what, const KeyTable& table)
{
    if (!block.isObject()) throw DefinitionError(string("Invalid ") + what + " entry (an object is expected)");
    for (auto& m : block.members())
        if (!dispatch(table, json::lower(m.first), m.second)) throw DefinitionError(string("Invalid ") + what + " parameter: " + m.first);
}

Setter toFloat(NNFloat& x)
{
    return [&x](const Value& v) { x = v.asFloat(); };
}

Setter toUInt(uint32_t& x)
{
    return [&x](const Value& v) { x = (uint32_t)v.asInt(); };
}

template <typename E> E lookup(const Value& v, const char* what, const std::vector<std::pair<const char*, E>>& names)
{
    const string s = json::lower(v.asString());
    for (auto& n : names)
        if (s == n.first) return n.second;
    throw DefinitionError(string("Invalid ") + what + ": " + v.asString());
}

void readExtent(const Value& v, uint32_t maxDims, uint32_t& x, uint32_t& y, uint32_t& z, uint32_t* w, uint32_t& dims, const string& layer)
{
    if (v.isArray()) {
        if (v.size() > maxDims) throw DefinitionError(">" + std::to_string(maxDims) + " dimensions detected in layer: " + layer);
        uint32_t* out[4] = {&x, &y, &z, w};
        for (size_t i = 0; i < v.size(); i++)
            if (out[i]) *out[i] = (uint32_t)v[i].asInt();
        dims = (uint32_t)v.size();
    } else {
        x = (uint32_t)v.asInt();
        dims = 1;
    }
}

void readLayer(const Value& layer, size_t position, size_t count, NNNetworkDescriptor& nd, std::set<string>& namesSeen,
               const vector<NNDataSetBase*>& vDataSet)
{
    if (!layer.isObject()) throw DefinitionError("layer " + std::to_string(position) + " is not an object");
    NNLayerDescriptor ld;
    ld._kind = (position == 0) ? NNLayer::Kind::Input : (position + 1 == count) ? NNLayer::Kind::Output : NNLayer::Kind::Hidden;
    ld._type = NNLayer::Type::FullyConnected;

    // kind and type decide which of the other keys are legal, so they are read first
    for (auto& m : layer.members()) {
        const string key = json::lower(m.first);
        if (key == "kind")
            ld._kind = lookup<NNLayer::Kind>(m.second, "layer kind",
                                             {{"input", NNLayer::Kind::Input}, {"hidden", NNLayer::Kind::Hidden},
                                              {"target", NNLayer::Kind::Target}, {"output", NNLayer::Kind::Output}});
        else if (key == "type")
            ld._type = lookup<NNLayer::Type>(m.second, "layer type",
                                             {{"fullyconnected", NNLayer::Type::FullyConnected},
                                              {"convolutional", NNLayer::Type::Convolutional}, {"pooling", NNLayer::Type::Pooling}});
    }
    if (ld._type != NNLayer::Type::FullyConnected) ld._bDimensionsProvided = false;
    ld._name = NNLayer::_sKindMap[ld._kind] + std::to_string(nd._vLayerDescriptor.size());

    const bool bInput = ld._kind == NNLayer::Kind::Input, bHidden = ld._kind == NNLayer::Kind::Hidden,
               bOutput = ld._kind == NNLayer::Kind::Output;
    bool bAutoSize = false, bSource = false;
    vector<NNWeightDescriptor> vShared;

    KeyTable any = {
        {"name",
         [&](const Value& v) {
             ld._name = v.asString();
             if (!namesSeen.insert(ld._name).second) throw DefinitionError("Duplicate layer name detected: " + ld._name);
         }},
        {"sparse", [&](const Value& v) { if (v.asBool()) ld._attributes |= NNLayer::Attributes::Sparse; }},
        {"n",
         [&](const Value& v) {
             if (v.isString()) {
                 // the only legal string is "auto" (not for hidden layers); other strings are ignored as upstream does
                 if (json::lower(v.asString()) == "auto") {
                     if (bHidden) throw DefinitionError("Illegal attempt to use auto for hidden layer: " + ld._name);
                     bAutoSize = true;
                 }
             } else
                 readExtent(v, 4, ld._Nx, ld._Ny, ld._Nz, &ld._Nw, ld._dimensions, ld._name);
         }},
        {"pdropout", toFloat(ld._pDropout)},
    };
    auto readKernel = [&](const Value& v, bool stride) {
        uint32_t x = 1, y = 1, z = 1, d = 1;
        readExtent(v, 3, x, y, z, nullptr, d, ld._name);
        if (stride) {
            ld._kernelStrideX = x, ld._kernelStrideY = y, ld._kernelStrideZ = z;
        } else {
            ld._kernelX = x, ld._kernelY = y, ld._kernelZ = z, ld._kernelDimensions = d;
        }
    };
    KeyTable notInput = {
        {"source",
         [&](const Value& v) {
             for (size_t i = 0; i < v.size(); i++) ld._vSource.push_back(v[i].asString());
             bSource = bSource || v.size() > 0;
         }},
        {"kernel", [&](const Value& v) { readKernel(v, false); }},
        {"kernelstride", [&](const Value& v) { readKernel(v, true); }},
    };
    KeyTable hidden = {
        {"batchnormalization", [&](const Value& v) { if (v.asBool()) ld._attributes |= NNLayer::Attributes::BatchNormalization; }},
        {"sparsenesspenalty",
         [&](const Value& v) {
             readBlock(v, ("sparseness penalty for hidden layer " + ld._name).c_str(),
                       {{"p", toFloat(ld._sparsenessPenalty_p)}, {"beta", toFloat(ld._sparsenessPenalty_beta)}});
         }},
    };
    KeyTable pooling = {
        {"function",
         [&](const Value& v) {
             ld._poolingFunction = lookup<PoolingFunction>(
                 v, ("pooling function for pooling layer " + ld._name).c_str(),
                 {{"max", PoolingFunction::Max}, {"maxout", PoolingFunction::Maxout}, {"dotproduct", PoolingFunction::DotProduct},
                  {"cosine", PoolingFunction::Cosine}, {"average", PoolingFunction::Average}, {"lrn", PoolingFunction::LRN},
                  {"localresponsenormalization", PoolingFunction::LRN}});
         }},
    };
    KeyTable computed = {
        {"skip", [&](const Value& v) { for (size_t i = 0; i < v.size(); i++) ld._vSkip.push_back(v[i].asString()); }},
        {"activation",
         [&](const Value& v) {
             ld._activation = lookup<Activation>(
                 v, "layer activation",
                 {{"sigmoid", Activation::Sigmoid}, {"tanh", Activation::Tanh}, {"linear", Activation::Linear},
                  {"relu", Activation::RectifiedLinear}, {"rectifiedlinear", Activation::RectifiedLinear},
                  {"lrelu", Activation::LeakyRectifiedLinear}, {"leakyrectifiedlinear", Activation::LeakyRectifiedLinear},
                  {"elu", Activation::ExponentialLinear}, {"exponentiallinear", Activation::ExponentialLinear},
                  {"selu", Activation::ScaledExponentialLinear}, {"scaledexponentiallinear", Activation::ScaledExponentialLinear},
                  {"softplus", Activation::SoftPlus}, {"softsign", Activation::SoftSign}, {"softmax", Activation::SoftMax},
                  {"relumax", Activation::RELUMax}, {"linearmax", Activation::LinearMax}});
         }},
        {"reluslope", toFloat(ld._RELUSlope)},
        {"slope", toFloat(ld._RELUSlope)},
        {"elualpha", toFloat(ld._ELUAlpha)},
        {"selulambda", toFloat(ld._SELULambda)},
        {"weightnorm", toFloat(ld._weightNorm)},
        {"deltanorm", toFloat(ld._deltaNorm)},
        {"weightinit",
         [&](const Value& v) {
             readBlock(v, "weight initialization",
                       {{"scheme",
                         [&](const Value& s) {
                             ld._weightInit = lookup<WeightInitialization>(
                                 s, "weight initialization scheme",
                                 {{"xavier", Xavier}, {"caffexavier", CaffeXavier}, {"gaussian", Gaussian}, {"uniform", Uniform},
                                  {"unitball", UnitBall}, {"constant", Constant}, {"selu", SELU}});
                         }},
                        {"scale", toFloat(ld._weightInitScale)},
                        {"bias", toFloat(ld._biasInit)}});
         }},
        {"sharedweights",
         [&](const Value& v) {
             for (size_t i = 0; i < v.size(); i++) {
                 NNWeightDescriptor share;
                 readBlock(v[i], "shared weight",
                           {{"sourceinputlayer", [&](const Value& s) { share._sourceInputLayer = s.asString(); }},
                            {"sourceoutputlayer", [&](const Value& s) { share._sourceOutputLayer = s.asString(); }},
                            {"inputlayer", [&](const Value& s) { share._inputLayer = s.asString(); }},
                            {"transposed", [&](const Value& s) { share._bTransposed = s.asBool(); }}});
                 share._bShared = true;
                 vShared.push_back(share);
             }
         }},
    };
    KeyTable withData = {{"dataset", [&](const Value& v) { ld._dataSet = v.asString(); }}};

    for (auto& m : layer.members()) {
        const string key = json::lower(m.first);
        if (key == "kind" || key == "type") continue;
        bool known = dispatch(any, key, m.second);
        if (!known && !bInput) known = dispatch(notInput, key, m.second);
        if (!known && bHidden) known = dispatch(hidden, key, m.second);
        if (!known && (bHidden || bOutput)) {
            if (ld._type == NNLayer::Type::Pooling) known = dispatch(pooling, key, m.second);
            if (!known) known = dispatch(computed, key, m.second);
        }
        if (!known && (bInput || bOutput)) known = dispatch(withData, key, m.second);
        if (!known) throw DefinitionError("Unknown neural network layer field: " + key);
    }

    if (bAutoSize) {
        const NNDataSetBase* found = nullptr;
        for (auto p : vDataSet)
            if (p && p->_name == ld._dataSet) found = p;
        if (!found) throw DefinitionError("Unable to find data set " + ld._dataSet + " to determine dimensions for layer: " + ld._name);
        ld._Nx = found->_width;
        ld._Ny = found->_height;
        ld._Nz = found->_length;
        ld._dimensions = found->_dimensions;
    }

    if (!bSource && !bInput) {
        if (nd._vLayerDescriptor.empty()) throw DefinitionError("Layer " + ld._name + " has no source and no layer before it");
        ld._vSource.push_back(nd._vLayerDescriptor.back()._name);
    }

    const bool bDot = ld._poolingFunction == PoolingFunction::DotProduct || ld._poolingFunction == PoolingFunction::Cosine;
    if (ld._type == NNLayer::Type::Pooling && bDot) {
        if (ld._vSource.size() < 2) throw DefinitionError("Dot product layer " + ld._name + " must have 2 or more sources");
        ld._Nx = (uint32_t)ld._vSource.size() - 1;
        ld._Ny = ld._Nz = 1;
        ld._dimensions = 1;
    }

    if (ld._type != NNLayer::Type::Pooling) {
        size_t sharedUsed = 0;
        for (auto& src : ld._vSource) {
            NNWeightDescriptor wd;
            wd._inputLayer = src;
            wd._outputLayer = ld._name;
            wd._norm = ld._weightNorm;
            for (auto& s : vShared) {
                if (s._inputLayer != src) continue;
                wd._bShared = true;
                wd._bTransposed = s._bTransposed;
                wd._sourceInputLayer = s._sourceInputLayer;
                wd._sourceOutputLayer = s._sourceOutputLayer;
                sharedUsed++;
                break;
            }
            nd._vWeightDescriptor.push_back(wd);
        }
        if (sharedUsed < vShared.size()) throw DefinitionError("Unable to locate all shared weights");
    }

    if (ld._dimensions < ld._kernelDimensions) ld._bDimensionsProvided = false;
    nd._vLayerDescriptor.push_back(ld);
}

void readNetwork(const Value& root, NNNetworkDescriptor& nd, const vector<NNDataSetBase*>& vDataSet)
{
    if (!root.isObject()) throw DefinitionError("the document is not an object");
    std::set<string> namesSeen;
    NNFloat maxoutK = (NNFloat)nd._maxout_k;
    Setter smce = [&](const Value& v) {
        readBlock(v, "ScaledMarginalCrossentropy",
                  {{"onescale", toFloat(nd._SMCE_oneScale)}, {"zeroscale", toFloat(nd._SMCE_zeroScale)},
                   {"onetarget", toFloat(nd._SMCE_oneTarget)}, {"zerotarget", toFloat(nd._SMCE_zeroTarget)}});
    };
    Setter lrn = [&](const Value& v) {
        readBlock(v, "LocalResponseNormalization",
                  {{"k", toFloat(nd._LRN_k)}, {"n", toUInt(nd._LRN_n)}, {"alpha", toFloat(nd._LRN_alpha)}, {"beta", toFloat(nd._LRN_beta)}});
    };
    KeyTable top = {
        {"version",
         [&](const Value& v) {
             if (v.asFloat() < 0.6999f) throw DefinitionError("version " + std::to_string(v.asFloat()) + " (must be at least 0.7)");
         }},
        {"name", [&](const Value& v) { nd._name = v.asString(); }},
        {"kind",
         [&](const Value& v) {
             nd._kind = lookup<NNNetwork::Kind>(v, "network kind",
                                                {{"feedforward", NNNetwork::Kind::FeedForward}, {"autoencoder", NNNetwork::Kind::AutoEncoder}});
         }},
        {"weightsdata", [&](const Value& v) { (void)v.asString(); }},   // named upstream, never read there either
        {"lrn", lrn},
        {"localresponsenormalization", lrn},
        {"maxout", [&](const Value& v) { readBlock(v, "MaxOut", {{"k", toFloat(maxoutK)}}); }},
        {"sparsenesspenalty",
         [&](const Value& v) {
             readBlock(v, "SparsenessPenalty", {{"p", toFloat(nd._sparsenessPenalty_p)}, {"beta", toFloat(nd._sparsenessPenalty_beta)}});
         }},
        {"denoising", [&](const Value& v) { readBlock(v, "Denoising", {{"p", toFloat(nd._denoising_p)}}); }},
        {"deltaboost",
         [&](const Value& v) { readBlock(v, "DeltaBoost", {{"one", toFloat(nd._deltaBoost_one)}, {"zero", toFloat(nd._deltaBoost_zero)}}); }},
        {"scaledmarginalcrossentropy", smce},
        {"datascaledmarginalcrossentropy", smce},
        {"shuffleindices", [&](const Value& v) { nd._bShuffleIndices = v.asBool(); }},
        {"reluslope", toFloat(nd._RELUSlope)},
        {"slope", toFloat(nd._RELUSlope)},
        {"elualpha", toFloat(nd._ELUAlpha)},
        {"selulambda", toFloat(nd._SELULambda)},
        {"decay", toFloat(nd._decay)},
        {"errorfunction",
         [&](const Value& v) {
             nd._errorFunction = lookup<ErrorFunction>(
                 v, "error function",
                 {{"l1", ErrorFunction::L1}, {"l2", ErrorFunction::L2}, {"l2hinge", ErrorFunction::L2Hinge}, {"hinge", ErrorFunction::Hinge},
                  {"crossentropy", ErrorFunction::CrossEntropy}, {"cross entropy", ErrorFunction::CrossEntropy},
                  {"scaledmarginalcrossentropy", ErrorFunction::ScaledMarginalCrossEntropy},
                  {"datascaledmarginalcrossentropy", ErrorFunction::DataScaledMarginalCrossEntropy}});
         }},
        {"layers",
         [&](const Value& v) {
             // one layer may be given without the surrounding array
             const size_t count = v.isArray() ? v.size() : 1;
             for (size_t i = 0; i < count; i++) readLayer(v.isArray() ? v[i] : v, i, count, nd, namesSeen, vDataSet);
         }},
    };
    for (auto& m : root.members())
        if (!dispatch(top, json::lower(m.first), m.second)) throw DefinitionError("Unknown neural network field: " + json::lower(m.first));
    nd._maxout_k = (uint32_t)maxoutK;

    nd._bSparsenessPenalty = nd._bSparsenessPenalty || nd._sparsenessPenalty_beta > (NNFloat)0.0;
    if (nd._denoising_p > (NNFloat)0.0) {
        nd._bDenoising = true;
        for (auto& l : nd._vLayerDescriptor)
            if (l._kind == NNLayer::Kind::Input && (l._attributes & NNLayer::Attributes::Sparse)) l._attributes |= NNLayer::Attributes::Denoising;
    }
    for (auto& l : nd._vLayerDescriptor) {
        if (std::isnan(l._RELUSlope)) l._RELUSlope = nd._RELUSlope;
        if (std::isnan(l._ELUAlpha)) l._ELUAlpha = nd._ELUAlpha;
        if (std::isnan(l._SELULambda)) l._SELULambda = nd._SELULambda;
    }
}

}  // namespace

bool LoadNNNetworkDescriptorJSON(const string& fname, NNNetworkDescriptor& nd, const vector<NNDataSetBase*>& vDataSet)
{
    json::Value root;
    string error;
    if (!json::parseFile(fname, root, error)) {
        printf("LoadNeuralNetworkJSON: Failed to parse JSON file: %s, error: %s\n", fname.c_str(), error.c_str());
        return false;
    }
    try {
        readNetwork(root, nd, vDataSet);
    } catch (std::exception& e) {
        printf("LoadNeuralNetworkJSON: %s\n", e.what());
        return false;
    }
    return true;
}

NNNetwork* LoadNeuralNetworkJSON(const string& fname, const uint32_t batch, const vector<NNDataSetBase*>& vDataSet)
{
    NNNetworkDescriptor nd;
    if (!LoadNNNetworkDescriptorJSON(fname, nd, vDataSet)) return NULL;
    cout << "LoadNeuralNetworkJSON: network " << nd._name << ", " << nd._vLayerDescriptor.size() << " layers, "
         << nd._vWeightDescriptor.size() << " weight sets" << endl;
    return CreateNeuralNetwork(nd, batch);
}
