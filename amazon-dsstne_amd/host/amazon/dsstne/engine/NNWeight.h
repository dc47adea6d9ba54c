// NNWeight.h — weights and biases of one fully connected connection (public surface of the reference's engine/NNWeight.h).
// W is [input stride][output stride] fp32 row-major, bias is [output stride]; no gradient or velocity buffers exist here.
#ifndef DSSTNE_AMD_NNWEIGHT_H
#define DSSTNE_AMD_NNWEIGHT_H

#include "GpuTypes.h"
#include "NNDefs.h"

class NNLayer;
class NNNetwork;

class NNWeight {
public:
    enum Transform { Convolution, Linear };

private:
    friend class NNNetwork;
    friend class NNLayer;

    NNLayer& _inputLayer;
    NNLayer& _outputLayer;
    const bool _bShared;          // uses another connection's matrix
    const bool _bTransposed;      // ... read as its transpose
    Transform _transform;
    bool _bLocked;
    NNWeight* _pSharedWeight;
    uint32_t _sharingCount;
    uint32_t _dimensionality;
    uint64_t _width;              // output units
    uint64_t _height;             // input units
    uint64_t _length;
    uint64_t _depth;
    uint64_t _breadth;
    uint64_t _size;
    uint64_t _biasSize;
    uint64_t _localSize;
    uint64_t _localBiasSize;
    NNFloat _norm;
    vector<NNFloat> _vWeight;
    vector<NNFloat> _vBias;
    unique_ptr<GpuBuffer<NNFloat>> _pbWeight;
    unique_ptr<GpuBuffer<NNFloat>> _pbBias;
    // NNNetwork::SetSplitProducts: the weights as three planes of bf16 (dsx_fc_split) for the dense kernel that forms its fp32
    // products from bf16 matrix instructions; one set per orientation in which layers use the matrix ([0]: stored [k][n],
    // [1]: stored [n][k]), built on first use and again after CopyWeights / SetWeights / Randomize / a load from file.
    unique_ptr<GpuBuffer<uint32_t>> _pbSplit[2];
    bool _bSplitValid[2] = {false, false};
    const void* SplitPlanes(bool bTransposed, uint32_t k, uint32_t n);
    void InvalidateSplit() { _bSplitValid[0] = _bSplitValid[1] = false; }

    NNWeight(NNLayer& inputLayer, NNLayer& outputLayer, bool bShared = false, bool bTransposed = false, bool bLocked = false,
             NNFloat maxNorm = 0.0f);
    ~NNWeight();
    NNFloat* GetWeightBuffer() { return _pbWeight ? _pbWeight->_pDevData : NULL; }
    // Starting values by the output layer's scheme (engine/NNWeight.cpp:500-561); biases start at biasInit.
    void Randomize();
    uint64_t GetBufferSize() { return _localSize; }

public:
    bool CopyWeights(const NNWeight* pWeight);
    bool SetWeights(const vector<NNFloat>& vWeight);
    bool SetBiases(const vector<NNFloat>& vBias);
    bool GetWeights(vector<NNFloat>& vWeight);
    bool GetBiases(vector<NNFloat>& vBias);
    bool GetDimensions(vector<uint64_t>& dimensions);
    bool SetNorm(NNFloat norm) { _norm = norm; return true; }
};

struct NNWeightDescriptor {
    string _inputLayer;
    string _outputLayer;
    uint64_t _width;
    uint64_t _height;
    uint64_t _length;
    uint64_t _depth;
    uint64_t _breadth;
    vector<NNFloat> _vWeight;
    vector<NNFloat> _vBias;
    bool _bShared;
    bool _bTransposed;
    bool _bLocked;
    NNFloat _norm;
    string _sourceInputLayer;
    string _sourceOutputLayer;

    NNWeightDescriptor();
};

#endif
