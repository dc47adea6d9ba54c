// NNWeight.cpp — fully connected weights and biases (reference: engine/NNWeight.cpp:289-479 constructor, 938-1057 setters and
// getters).  Only the inference state exists: the matrix, the bias vector and their host shadows.
#include <cinttypes>
#include <cmath>

#include "amazon/dsstne/engine/NNTypes.h"

NNWeightDescriptor::NNWeightDescriptor()
    : _width(1), _height(1), _length(1), _depth(1), _breadth(1), _bShared(false), _bTransposed(false), _bLocked(false), _norm(0.0f)
{
}

NNWeight::NNWeight(NNLayer& inputLayer, NNLayer& outputLayer, bool bShared, bool bTransposed, bool bLocked, NNFloat norm)
    : _inputLayer(inputLayer), _outputLayer(outputLayer), _bShared(bShared), _bTransposed(bTransposed), _transform(Linear),
      _bLocked(bLocked), _pSharedWeight(NULL), _sharingCount(1), _dimensionality(2), _width(1), _height(1), _length(1), _depth(1),
      _breadth(1), _size(0), _biasSize(0), _localSize(0), _localBiasSize(0), _norm(norm)
{
    inputLayer._vOutgoingLayer.push_back(&outputLayer);
    outputLayer._vIncomingLayer.push_back(&inputLayer);
    inputLayer._vOutgoingWeight.push_back(this);
    outputLayer._vIncomingWeight.push_back(this);

    if (outputLayer._type != NNLayer::Type::FullyConnected) {
        printf("NNWeight::NNWeight: only fully connected layers are supported by this build (layer %s).\n", outputLayer._name.c_str());
        getGpu().Shutdown();
        exit(-1);
    }

    // W[input unit][output unit], output unit contiguous
    _width = outputLayer._stride;
    _height = inputLayer._stride;
    _localSize = _width * _height * _length * _depth * _breadth;
    _localBiasSize = outputLayer._localStride;
    _size = (uint64_t)outputLayer._stride * inputLayer._stride * _length * _depth * _breadth;
    _biasSize = outputLayer._stride;

    if (!_bShared) {
        printf("NNWeight::NNWeight: Allocating %" PRIu64 " bytes (%" PRIu64 ", %" PRIu64 ") for fully connected weights between layers %s and %s\n",
               _localSize * sizeof(NNFloat), _width, _height, inputLayer._name.c_str(), outputLayer._name.c_str());
        _vWeight.resize(_localSize);
        _pbWeight.reset(new GpuBuffer<NNFloat>(_localSize));
    }
    _vBias.resize(_localBiasSize);
    _pbBias.reset(new GpuBuffer<NNFloat>(_localBiasSize));
}

NNWeight::~NNWeight() {}

namespace {
// Counter-based stream: value i of a connection depends only on the process seed, the two layer names and i, so a
// network gets the same starting weights however its connections are ordered.  (The reference draws from cuRAND's
// default generator, whose stream is not reproduced here.)
struct WeightStream {
    uint64_t key;
    WeightStream(unsigned long seed, const string& in, const string& out) : key(0x9E3779B97F4A7C15ull ^ (uint64_t)seed)
    {
        for (unsigned char c : in) key = (key ^ c) * 0x100000001B3ull;
        key = (key ^ 0xFFu) * 0x100000001B3ull;
        for (unsigned char c : out) key = (key ^ c) * 0x100000001B3ull;
    }
    uint64_t bits(uint64_t i) const
    {
        uint64_t z = key + (i + 1) * 0x9E3779B97F4A7C15ull;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    // in (0, 1], like the generator the reference uses
    float uniform(uint64_t i) const { return (float)((bits(i) >> 40) + 1) * (1.0f / 16777216.0f); }
    float normal(uint64_t i) const
    {
        const uint64_t pair = i >> 1;
        const float r = sqrtf(-2.0f * logf(uniform(2 * pair))), a = 6.28318530717958647692f * uniform(2 * pair + 1);
        return (i & 1) ? r * sinf(a) : r * cosf(a);
    }
};
}  // namespace

void NNWeight::Randomize()
{
    if (!_bShared) {
        const WeightStream rng(getGpu()._randomSeed, _inputLayer._name, _outputLayer._name);
        const NNFloat s = _outputLayer._weightInitScale;
        const NNFloat nOut = (NNFloat)_outputLayer._stride, nIn = (NNFloat)_inputLayer._stride;
        NNFloat scale = 0.0f, shift = 0.0f, sigma = 0.0f;
        bool bNormal = false;
        switch (_outputLayer._weightInit) {
        case CaffeXavier:   // uniform in ±s·sqrt(3 / n_out)
            scale = s * 2.0f * sqrtf(3.0f / nOut);
            shift = 0.5f * scale;
            break;
        case Xavier:        // uniform in ±s·sqrt(6 / (n_out + n_in)) / 2, as the reference scales it
            scale = s * sqrtf(6.0f / (nOut + nIn));
            shift = 0.5f * scale;
            break;
        case Uniform:       // uniform in ±s
            scale = 2.0f * s;
            shift = 0.5f * scale;
            break;
        case UnitBall:      // uniform in (0, s]
            scale = s;
            break;
        case Gaussian:      // N(0, s)
            bNormal = true;
            sigma = s;
            break;
        case SELU:          // N(0, 1 / n_in)
            bNormal = true;
            sigma = 1.0f / nIn;
            break;
        case Constant:      // the reference's scale-and-shift step computes 0·scale − s here, so every weight is −s
            shift = s;
            break;
        }
        const uint64_t n = _vWeight.size();
        if (bNormal) {
            for (uint64_t i = 0; i < n; i++) _vWeight[i] = sigma * rng.normal(i);
        } else if (scale != 0.0f) {
            for (uint64_t i = 0; i < n; i++) _vWeight[i] = rng.uniform(i) * scale - shift;
        } else {
            std::fill(_vWeight.begin(), _vWeight.end(), -shift);
        }
        _pbWeight->Upload(_vWeight.data());
        InvalidateSplit();
    }
    std::fill(_vBias.begin(), _vBias.end(), _outputLayer._biasInit);
    _pbBias->Upload(_vBias.data());
}

bool NNWeight::CopyWeights(const NNWeight* pSrcWeight)
{
    NNWeight* pDstWeight = _bShared ? _pSharedWeight : this;
    if (!pSrcWeight) {
        printf("NNWeight::CopyWeights: Invalid weight pointer.\n");
        return false;
    }
    const NNWeight* pSrc = _bShared ? pSrcWeight->_pSharedWeight : pSrcWeight;
    if (!pSrc || (pSrc->_width != pDstWeight->_width) || (pSrc->_height != pDstWeight->_height) || (pSrc->_length != pDstWeight->_length)) {
        printf("NNWeight::CopyWeights: Mismatched weight dimensions.\n");
        return false;
    }
    pDstWeight->_vWeight = pSrc->_vWeight;
    _vBias = pSrcWeight->_vBias;
    if (pDstWeight->_pbWeight) pDstWeight->_pbWeight->Upload(pDstWeight->_vWeight.data());
    pDstWeight->InvalidateSplit();
    if (_pbBias) _pbBias->Upload(_vBias.data());
    return true;
}

bool NNWeight::SetWeights(const vector<NNFloat>& vWeight)
{
    NNWeight* pWeight = _bShared ? _pSharedWeight : this;
    if (vWeight.size() < pWeight->_vWeight.size()) {
        printf("NNWeight::SetWeights: Input vector smaller than weight vector.\n");
        return false;
    }
    std::copy(vWeight.begin(), vWeight.begin() + pWeight->_vWeight.size(), pWeight->_vWeight.begin());
    if (pWeight->_pbWeight) pWeight->_pbWeight->Upload(pWeight->_vWeight.data());
    pWeight->InvalidateSplit();
    return true;
}

// The matrix as dsx_fc_forward_split wants it, for a layer that multiplies [batch x k] inputs into n units: column j of the
// product's W is row j of the planes.  Built on the calling lane's stream; every lane waits for it once (dsx_sync), after that
// the planes are only read.
const void* NNWeight::SplitPlanes(bool bTransposed, uint32_t k, uint32_t n)
{
    const int o = bTransposed ? 1 : 0;
    if (!_bSplitValid[o]) {
        const size_t words = (size_t)(dsx_fc_split_bytes(n, k) / sizeof(uint32_t));
        if (!_pbSplit[o] || _pbSplit[o]->_length < words) _pbSplit[o].reset(new GpuBuffer<uint32_t>(words));
        dsxFatal(dsx_fc_split(_pbWeight->_pDevData, bTransposed ? k : n, bTransposed ? 0 : 1, n, k, _pbSplit[o]->_pDevData),
                 "NNWeight::SplitPlanes");
        dsxFatal(dsx_sync(), "NNWeight::SplitPlanes");
        _bSplitValid[o] = true;
    }
    return _pbSplit[o]->_pDevData;
}

bool NNWeight::SetBiases(const vector<NNFloat>& vBias)
{
    if (vBias.size() < _vBias.size()) {
        printf("NNWeight::SetBiases: Input vector smaller than bias vector.\n");
        return false;
    }
    std::copy(vBias.begin(), vBias.begin() + _vBias.size(), _vBias.begin());
    if (_pbBias) _pbBias->Upload(_vBias.data());
    return true;
}

bool NNWeight::GetWeights(vector<NNFloat>& vWeight)
{
    if (vWeight.size() < _vWeight.size()) vWeight.resize(_vWeight.size());
    if (_pbWeight)
        _pbWeight->Download(vWeight.data());
    else
        vWeight = _vWeight;
    return true;
}

bool NNWeight::GetBiases(vector<NNFloat>& vBias)
{
    if (vBias.size() < _vBias.size()) vBias.resize(_vBias.size());
    if (_pbBias)
        _pbBias->Download(vBias.data());
    else
        vBias = _vBias;
    return true;
}

bool NNWeight::GetDimensions(vector<uint64_t>& dimensions)
{
    if (_dimensionality < 2 || _dimensionality > 5) {
        printf("NNWeight::GetDimensions: _dimensionality = %u\n", _dimensionality);
        return false;
    }
    dimensions.push_back(_width);
    dimensions.push_back(_height);
    if (_dimensionality >= 3) dimensions.push_back(_length);
    if (_dimensionality >= 4) dimensions.push_back(_depth);
    if (_dimensionality == 5) dimensions.push_back(_breadth);
    return true;
}
