// NNLayer.h — one layer of a feed-forward network (public surface of the reference's engine/NNLayer.h:211-263).
// Only fully connected layers run in this build; activations live in a [batch][stride] fp32 buffer in HBM, and a
// fast-sparse input layer owns no buffer at all (its dataset feeds the next layer's SpMM directly).
#ifndef DSSTNE_AMD_NNLAYER_H
#define DSSTNE_AMD_NNLAYER_H

#include "GpuTypes.h"
#include "NNDefs.h"

struct NNLayerDescriptor;
struct NNDataSetBase;
class NNWeight;
class NNNetwork;

class NNLayer {
public:
    friend class NNNetwork;
    friend class NNWeight;

    enum Kind { Input, Hidden, Output, Target };
    static std::map<Kind, string> _sKindMap;

    enum Type { FullyConnected, Convolutional, Pooling };
    static std::map<Type, string> _sTypeMap;

    enum Attributes { None = 0x0, Sparse = 0x1, Denoising = 0x2, BatchNormalization = 0x4 };

    enum Parallelization { Data, Model, Serial };

private:
    const string _name;
    const Kind _kind;
    const Type _type;
    const uint32_t _attributes;
    string _dataSet;
    NNDataSetBase* _pDataSet;
    vector<string> _vSource;
    vector<string> _vSkip;
    uint32_t _Nx, _Ny, _Nz, _Nw;
    uint32_t _stride;
    uint32_t _localStride;
    uint32_t _maxLocalStride;
    uint32_t _batch;
    uint32_t _localBatch;
    uint32_t _dimensions;
    uint32_t _minX, _maxX;
    NNFloat _RELUSlope, _ELUAlpha, _SELULambda;
    const Activation _activation;
    const NNFloat _pDropout;
    const WeightInitialization _weightInit;     // how weights into this layer start when a definition supplies none
    const NNFloat _weightInitScale;
    const NNFloat _biasInit;
    bool _bSparse;
    bool _bFastSparse;
    bool _bDirty;
    vector<NNLayer*> _vIncomingLayer;
    vector<NNWeight*> _vIncomingWeight;
    vector<NNLayer*> _vOutgoingLayer;
    vector<NNWeight*> _vOutgoingWeight;
    vector<NNLayer*> _vIncomingSkip;
    vector<NNLayer*> _vOutgoingSkip;
    unique_ptr<GpuBuffer<NNFloat>> _pbUnit;
    // Maxima of the 64-unit segments of every row of _pbUnit, left by the dense kernel that produced the current batch
    // (_segWidth == 0: none): NNNetwork::CalculateTopK then reads only the segments that can hold a result.
    unique_ptr<GpuBuffer<NNFloat>> _pbSegMax;
    uint32_t _segWidth = 0;
    // With several lanes (NNNetwork::SetLanes) every layer has one set of the three members above (and of the two deferral
    // members below) per lane: the batches before the current one may still be running on the other lanes' streams.  The
    // names above always denote the current batch's buffers; SwitchLane parks them under the lane they belong to and takes
    // out the set of the lane the next batch runs on.
    struct LaneSet {
        unique_ptr<GpuBuffer<NNFloat>> unit;
        unique_ptr<GpuBuffer<NNFloat>> segMax;
        unique_ptr<GpuBuffer<uint32_t>> splitInput;
        bool splitInputFresh = false;
        uint32_t segWidth = 0;
        bool deferred = false;
        uint32_t deferredBatch = 0;
    };
    LaneSet _parked[DSX_MAX_LANES];
    uint32_t _currentLane = 0;
    uint32_t _lanes = 1;
    // A wide output layer that feeds nothing but a top-K is not computed by the forward pass: NNNetwork::CalculateTopK /
    // CalculateFilteredTopK then run the layer and the top-K in one call that never stores the layer's result (dsx_fc_topk), and
    // whoever asks for the units themselves (NNNetwork::GetUnitBuffer, GetUnits) has them computed at that moment (Materialise).
    // _deferred: the units of the current batch have not been computed yet; _deferredBatch: its rows.
    bool _bDeferOutput = true;   // NNNetwork::SetDeferredOutput
    // NNNetwork::SetSplitProducts: this layer's input as bf16 planes (dsx_fc_split), written before the layer's kernel on the
    // same stream; one buffer per lane, like the units.
    bool _bSplitProducts = false;
    uint32_t _splitMinTiles = 0;
    unique_ptr<GpuBuffer<uint32_t>> _pbSplitInput;
    bool _bSplitInputFresh = false;   // the layer before this one wrote the planes of the current batch itself (dsx_fc_forward_planes)
    void* SplitInputBuffer();         // this lane's buffer for them, allocated on first use
    bool UseSplitProducts(uint32_t batch) const
    {
        if (!_bSplitProducts || _vIncomingLayer.empty()) return false;
        // (a plane of the kernel's operands stays below 4 GiB: 2 bytes x inputs padded to 16 x units padded to 256)
        const uint64_t plane = 2ull * ((_vIncomingLayer[0]->_stride + 15) / 16 * 16) * ((uint64_t)(_localStride + 255) / 256 * 256);
        return plane < (1ull << 32) && (uint64_t)((batch + 127) / 128) * ((_localStride + 127) / 128) >= _splitMinTiles;
    }
    // Z = act(bias + X.W) of a single-source layer through dsx_fc_split + dsx_fc_forward_split (segment maxima on request).
    void ForwardSplit(uint32_t batch, NNFloat* pSegMax, uint32_t* pSegWidth);
    const void* SplitInput(uint32_t batch);   // the source layer's units of this batch as planes (this lane's buffer)
    bool _deferred = false;
    uint32_t _deferredBatch = 0;
    void Materialise();
    void SwitchLane(uint32_t lane)
    {
        if (lane == _currentLane) return;
        LaneSet& mine = _parked[_currentLane];
        mine.unit.swap(_pbUnit);
        mine.segMax.swap(_pbSegMax);
        mine.splitInput.swap(_pbSplitInput);
        mine.splitInputFresh = _bSplitInputFresh;
        mine.segWidth = _segWidth;
        mine.deferred = _deferred;
        mine.deferredBatch = _deferredBatch;
        LaneSet& next = _parked[lane];
        _pbUnit.swap(next.unit);
        _pbSegMax.swap(next.segMax);
        _pbSplitInput.swap(next.splitInput);
        _bSplitInputFresh = next.splitInputFresh;
        _segWidth = next.segWidth;
        _deferred = next.deferred;
        _deferredBatch = next.deferredBatch;
        _currentLane = lane;
    }
    int32_t _priority;

    NNLayer(NNLayerDescriptor& l, uint32_t batch);
    ~NNLayer();
    void Allocate(bool validate);
    void Deallocate();
    void SetBatch(uint32_t batch);
    void RefreshState(NNNetwork* pNetwork, TrainingMode trainingMode, bool validate);
    void LoadPredictionBatch(uint32_t position, uint32_t batch);
    void ForwardPropagate(uint32_t position, uint32_t batch, bool bTraining = false);
    void ForwardPropagateFullyConnected(uint32_t position, uint32_t batch, bool bTraining);
    void CalculateActivation(uint32_t batch);
    NNFloat* GetIncomingUnitBuffer() { return _pbUnit ? _pbUnit->_pDevData : NULL; }
    NNFloat* GetUnitBuffer() { return _pbUnit ? _pbUnit->_pDevData : NULL; }
    uint64_t GetBufferSize() { return (uint64_t)_batch * (uint64_t)_stride; }

public:
    const string& GetName() const;
    const string& GetDataSetName() const;
    Kind GetKind() const;
    Type GetType() const;
    uint32_t GetAttributes() const;
    NNDataSetBase* GetDataSet() const;
    uint32_t GetNumDimensions() const;
    tuple<uint32_t, uint32_t, uint32_t, uint32_t> GetDimensions() const;
    tuple<uint32_t, uint32_t, uint32_t, uint32_t> GetLocalDimensions() const;
    Activation GetActivation() const { return _activation; }
    bool GetUnits(vector<NNFloat>& vUnit);
    bool GetUnits(NNFloat* pUnit);
    bool SetUnits(const vector<NNFloat>& vUnit);
};

ostream& operator<<(ostream& out, NNLayer::Kind& k);
ostream& operator<<(ostream& out, NNLayer::Type& t);

struct NNLayerDescriptor {
    string _name;
    NNLayer::Kind _kind;
    NNLayer::Type _type;
    PoolingFunction _poolingFunction;
    string _dataSet;
    vector<string> _vSource;
    vector<string> _vSkip;
    uint32_t _Nx, _Ny, _Nz, _Nw;
    uint32_t _dimensions;
    bool _bDimensionsProvided;
    WeightInitialization _weightInit;
    NNFloat _weightInitScale;
    NNFloat _biasInit;
    uint32_t _kernelX, _kernelY, _kernelZ;
    uint32_t _kernelStrideX, _kernelStrideY, _kernelStrideZ;
    uint32_t _kernelPaddingX, _kernelPaddingY, _kernelPaddingZ;
    uint32_t _kernelDimensions;
    NNFloat _weightNorm;
    NNFloat _deltaNorm;
    NNFloat _pDropout;
    Activation _activation;
    NNFloat _sparsenessPenalty_p;
    NNFloat _sparsenessPenalty_beta;
    uint32_t _attributes;
    NNFloat _RELUSlope;
    NNFloat _ELUAlpha;
    NNFloat _SELULambda;
    NNLayerDescriptor();
};

#endif
