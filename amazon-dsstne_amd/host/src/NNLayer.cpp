// NNLayer.cpp — layer state and the single-device forward step (reference: engine/NNLayer.cpp:36-254 constructor, 587-680
// Allocate, 799-885 RefreshState, 894-908 LoadPredictionBatch, 994-1168 ForwardPropagateFullyConnected, 1646-1683
// CalculateActivation).
//
// The reference spends three kernels per layer (bias fill, product, activation).  Here a layer with one source and no skip
// connection is a single fused kernel: sparse Z + bias + activation for a fast-sparse input, or MFMA GEMM + bias +
// activation for a dense source.  Layers with several sources or skips fall back to the reference's step sequence.
#include <cinttypes>
#include <cmath>

#include "amazon/dsstne/engine/NNTypes.h"

std::map<NNLayer::Kind, string> NNLayer::_sKindMap = {{NNLayer::Kind::Input, "Input"}, {NNLayer::Kind::Hidden, "Hidden"},
                                                     {NNLayer::Kind::Output, "Output"}, {NNLayer::Kind::Target, "Target"}};
std::map<NNLayer::Type, string> NNLayer::_sTypeMap = {{NNLayer::Type::FullyConnected, "FullyConnected"},
                                                     {NNLayer::Type::Convolutional, "Convolutional"}, {NNLayer::Type::Pooling, "Pooling"}};

ostream& operator<<(ostream& out, NNLayer::Kind& k) { return out << NNLayer::_sKindMap[k]; }
ostream& operator<<(ostream& out, NNLayer::Type& t) { return out << NNLayer::_sTypeMap[t]; }

ostream& operator<<(ostream& out, const Activation& a)
{
    static const char* names[] = {"Sigmoid", "Tanh", "RectifiedLinear", "Linear", "ParametricRectifiedLinear", "SoftPlus", "SoftSign",
                                  "SoftMax", "RELUMax", "LinearMax", "ExponentialLinear", "LeakyRectifiedLinear", "ScaledExponentialLinear"};
    return out << (((unsigned)a < 13) ? names[(unsigned)a] : "Unknown");
}

NNLayerDescriptor::NNLayerDescriptor()
    : _kind(NNLayer::Kind::Hidden), _type(NNLayer::Type::FullyConnected), _poolingFunction(None), _Nx(1), _Ny(1), _Nz(1), _Nw(1),
      _dimensions(1), _bDimensionsProvided(true), _weightInit(Xavier), _weightInitScale((NNFloat)1.0), _biasInit((NNFloat)0.0), _kernelX(1),
      _kernelY(1), _kernelZ(1), _kernelStrideX(1), _kernelStrideY(1), _kernelStrideZ(1), _kernelPaddingX(0), _kernelPaddingY(0),
      _kernelPaddingZ(0), _kernelDimensions(1), _weightNorm((NNFloat)0.0), _deltaNorm((NNFloat)0.0), _pDropout((NNFloat)0.0),
      _activation(Activation::Sigmoid), _sparsenessPenalty_p((NNFloat)0.0), _sparsenessPenalty_beta((NNFloat)0.0),
      _attributes(NNLayer::Attributes::None), _RELUSlope(NAN), _ELUAlpha(NAN), _SELULambda(NAN)
{
}

NNLayer::NNLayer(NNLayerDescriptor& d, uint32_t batch)
    : _name(d._name), _kind(d._kind), _type(d._type), _attributes(d._attributes), _dataSet(d._dataSet), _pDataSet(NULL),
      _vSource(d._vSource), _vSkip(d._vSkip), _Nx(d._Nx), _Ny(d._Ny), _Nz(d._Nz), _Nw(d._Nw), _batch(batch), _localBatch(batch),
      _dimensions(d._dimensions), _RELUSlope(d._RELUSlope), _ELUAlpha(d._ELUAlpha), _SELULambda(d._SELULambda),
      _activation(d._activation), _pDropout(d._pDropout), _weightInit(d._weightInit), _weightInitScale(d._weightInitScale),
      _biasInit(d._biasInit), _bSparse(d._attributes & NNLayer::Attributes::Sparse), _bFastSparse(false),
      _bDirty(true), _priority(-1)
{
    _stride = _Nx * _Ny * _Nz * _Nw;
    _minX = 0;
    _maxX = _Nx;
    _localStride = _stride;
    _maxLocalStride = _stride;
    if (d._attributes & NNLayer::Attributes::BatchNormalization) {
        printf("NNLayer::NNLayer: batch normalization is not supported by this build (layer %s).\n", _name.c_str());
        getGpu().Shutdown();
        exit(-1);
    }
}

NNLayer::~NNLayer() { Deallocate(); }

void NNLayer::Deallocate()
{
    _pbUnit.reset();
    _pbSegMax.reset();
    _pbSplitInput.reset();
    _segWidth = 0;
    _deferred = false;
    for (auto& set : _parked) set = LaneSet();
}

void NNLayer::SetBatch(uint32_t batch)
{
    if (batch != _batch) {
        _batch = batch;
        _localBatch = batch;
        _bDirty = true;
    }
}

void NNLayer::Allocate(bool validate)
{
    Deallocate();
    const uint64_t size = (uint64_t)_maxLocalStride * (uint64_t)_localBatch;
    // hidden and output layers, dense inputs and sparse inputs that cannot use the sparse-Z path own an activation buffer
    if (!_bSparse || !_bFastSparse || (_kind != Input) || (_bSparse && (_kind == Input) && validate)) {
        _pbUnit.reset(new GpuBuffer<NNFloat>(size));
        for (uint32_t lane = 0; lane < _lanes; lane++)
            if (lane != _currentLane) _parked[lane].unit.reset(new GpuBuffer<NNFloat>(size));
        printf("NNLayer::Allocate: Allocating %" PRIu64 " bytes (%u, %u) of unit data for layer %s", size * sizeof(NNFloat), _maxLocalStride, _localBatch,
               _name.c_str());
        if (_lanes > 1) printf(", %u times (one per lane)", _lanes);
        printf("\n");
    }
    _bDirty = false;
}

void NNLayer::RefreshState(NNNetwork* pNetwork, TrainingMode trainingMode, bool validate)
{
    (void)pNetwork;
    (void)trainingMode;
    if (_bDirty) {
        _bFastSparse = false;
        if ((_kind == Input) && (_pDataSet != NULL) && _bSparse) {
            if (_pDataSet->_sparseDensity > (NNFloat)0.1)
                printf("NNLayer::RefreshState: Sparse density per (%.2f) is too high to use fast sparse kernels on input layer %s\n",
                       _pDataSet->_sparseDensity, _name.c_str());
            else
                _bFastSparse = true;
        }
        Allocate(validate);
        if ((_kind != Hidden) && (_pDataSet != NULL)) _pDataSet->Shard(NNDataSetEnums::Model);
        _bDirty = false;
    }
}

void NNLayer::LoadPredictionBatch(uint32_t position, uint32_t batch)
{
    if (_kind == Input) {
        if (!_bSparse)
            _pDataSet->LoadInputUnit(position, batch, _localStride, _pbUnit->_pDevData);
        else if (!_bFastSparse)
            _pDataSet->LoadSparseInputUnit(position, batch, _localStride, _pbUnit->_pDevData);
    }
}

void NNLayer::ForwardPropagate(uint32_t position, uint32_t batch, bool bTraining)
{
    if (_type != FullyConnected) {
        printf("NNLayer::ForwardPropagate: layer %s is not fully connected; only fully connected layers run in this build.\n", _name.c_str());
        getGpu().Shutdown();
        exit(-1);
    }
    ForwardPropagateFullyConnected(position, batch, bTraining);
}

// Narrower layers are cheap to scan in full.
static const uint32_t kSegMaxMinWidth = 8192;
// From this width on the output layer is not stored but computed together with its top-K.  What the GEMM kernel's epilogue
// then does per 32 x 32 block depends on how many scores of the block reach the row's running k-th score: about
// 1024 * (k / columns seen so far + the filter's density).  In a 27,278-wide catalogue with top-10 and 144 own items per sample
// that is ten per block, every block takes the slow path and the fused call is no faster than storing the layer (measured:
// 95 us against 76 us for the GEMM alone); in a 1,000,000-wide one it is one block in three, and 16 GB of stores and loads go away.
static const uint32_t kDeferMinWidth = 131072;

void NNLayer::ForwardPropagateFullyConnected(uint32_t position, uint32_t batch, bool bTraining)
{
    (void)bTraining;
    if (_kind == Input) return;
    const size_t nIn = _vIncomingLayer.size();
    if (nIn > 4) {
        printf("NNLayer::ForwardPropagate: Too many input layers for network layer %s\n", _name.c_str());
        getGpu().Shutdown();
        exit(-1);
    }
    dsx_act_params params = {_RELUSlope, _ELUAlpha, _SELULambda};
    NNFloat* pUnit = GetIncomingUnitBuffer();
    _segWidth = 0;   // whatever described the previous batch no longer holds
    _deferred = false;

    // One source, no skips, elementwise activation: a single fused kernel.
    if (nIn == 1 && _vIncomingSkip.empty() && _activation != SoftMax) {
        NNLayer* src = _vIncomingLayer[0];
        NNWeight* w = _vIncomingWeight[0];
        NNWeight* wsrc = w->_bShared ? w->_pSharedWeight : w;
        if (src->_bFastSparse) {
            src->_pDataSet->CalculateSparseLayer(position, batch, _stride, wsrc->_pbWeight->_pDevData, w->_pbBias->_pDevData, _activation,
                                                 _RELUSlope, _ELUAlpha, _SELULambda, pUnit);
        } else if (_kind == Output && _localStride >= kSegMaxMinWidth) {
            // Wide output layer that feeds no other layer: what usually follows is a top-K, which can run together with the layer
            // without the layer's result ever being stored.  The layer is computed when somebody asks for it.
            if (_bDeferOutput && _localStride >= kDeferMinWidth && !w->_bTransposed && _vOutgoingLayer.empty() && _vOutgoingSkip.empty() &&
                dsx_fc_topk_supported(src->_stride, src->GetUnitBuffer(), (uint32_t)_activation, &params, NULL)) {
                if (dsx_fc_topk_flagged_for(wsrc->_pbWeight->_pDevData, 0)) {
                    // rows whose survivor lists filled up had to be recomputed one by one: this data (thousands of scores tied at the
                    // top of a row) is served better by the stored layer and the scanning top-K
                    printf("NNLayer::ForwardPropagate: scores of layer %s tie in their thousands; its result is stored from now on.\n", _name.c_str());
                    _bDeferOutput = false;
                } else {
                    _deferred = true;
                    _deferredBatch = batch;
                    return;
                }
            }
            _deferredBatch = batch;
            Materialise();
        } else if (UseSplitProducts(batch)) {
            ForwardSplit(batch, NULL, NULL);
        } else {
            // The only consumer of this layer forms its products from bf16 planes of its input: this layer's kernel writes them
            // along with its result (one launch less per batch than splitting the result afterwards).
            NNLayer* next = (_vOutgoingLayer.size() == 1 && _vOutgoingSkip.empty()) ? _vOutgoingLayer[0] : NULL;
            if (next && next->_vIncomingLayer.size() == 1 && next->_vIncomingLayer[0] == this && next->UseSplitProducts(batch)) {
                dsxFatal(dsx_fc_forward_planes(src->GetUnitBuffer(), src->_stride, wsrc->_pbWeight->_pDevData, w->_bTransposed ? 1 : 0,
                                               w->_pbBias->_pDevData, pUnit, _stride, batch, src->_stride, _localStride, (uint32_t)_activation,
                                               &params, next->SplitInputBuffer()),
                         "NNLayer::ForwardPropagate: GEMM failure");
                next->_bSplitInputFresh = true;
            } else
                dsxFatal(dsx_fc_forward(src->GetUnitBuffer(), src->_stride, wsrc->_pbWeight->_pDevData, w->_bTransposed ? 1 : 0,
                                        w->_pbBias->_pDevData, pUnit, _stride, batch, src->_stride, _localStride, 0, (uint32_t)_activation, &params),
                         "NNLayer::ForwardPropagate: GEMM failure");
        }
        return;
    }

    // General case, in the reference's order: bias sum, one product per source accumulated into z, skips, activation.
    NNFloat* bias[4] = {NULL, NULL, NULL, NULL};
    for (size_t i = 0; i < nIn; i++) bias[i] = _vIncomingWeight[i]->_pbBias->_pDevData;
    dsxFatal(dsx_clear_unit(pUnit, bias[0], bias[1], bias[2], bias[3], (uint32_t)nIn, _stride, batch), "NNLayer::ForwardPropagate: bias");
    for (size_t i = 0; i < nIn; i++) {
        NNLayer* src = _vIncomingLayer[i];
        NNWeight* w = _vIncomingWeight[i];
        NNWeight* wsrc = w->_bShared ? w->_pSharedWeight : w;
        if (src->_bFastSparse)
            src->_pDataSet->CalculateSparseZ(position, batch, _stride, wsrc->_pbWeight->_pDevData, pUnit, (NNFloat)1.0);
        else
            dsxFatal(dsx_fc_forward(src->GetUnitBuffer(), src->_stride, wsrc->_pbWeight->_pDevData, w->_bTransposed ? 1 : 0, NULL, pUnit,
                                    _stride, batch, src->_stride, _localStride, 1, DSX_ACT_LINEAR, &params),
                     "NNLayer::ForwardPropagate: GEMM failure");
    }
    for (auto l : _vIncomingSkip) dsxFatal(dsx_add_buffers(pUnit, l->GetUnitBuffer(), (uint64_t)batch * _stride), "NNLayer::ForwardPropagate: skip");
    CalculateActivation(batch);
}

// The wide output layer's own kernel: stores the layer's result and leaves segment maxima for the top-K that usually follows.
void NNLayer::Materialise()
{
    _deferred = false;
    NNLayer* src = _vIncomingLayer[0];
    NNWeight* w = _vIncomingWeight[0];
    NNWeight* wsrc = w->_bShared ? w->_pSharedWeight : w;
    dsx_act_params params = {_RELUSlope, _ELUAlpha, _SELULambda};
    const size_t need = (size_t)_batch * ((_localStride + 63) / 64);
    if (!_pbSegMax || _pbSegMax->_length < need) _pbSegMax.reset(new GpuBuffer<NNFloat>(need));
    if (UseSplitProducts(_deferredBatch)) {
        ForwardSplit(_deferredBatch, _pbSegMax->_pDevData, &_segWidth);
        return;
    }
    dsxFatal(dsx_fc_forward_segmax(src->GetUnitBuffer(), src->_stride, wsrc->_pbWeight->_pDevData, w->_bTransposed ? 1 : 0,
                                   w->_pbBias->_pDevData, GetIncomingUnitBuffer(), _stride, _deferredBatch, src->_stride, _localStride,
                                   (uint32_t)_activation, &params, _pbSegMax->_pDevData, &_segWidth),
             "NNLayer::ForwardPropagate: GEMM failure");
}

void NNLayer::ForwardSplit(uint32_t batch, NNFloat* pSegMax, uint32_t* pSegWidth)
{
    NNLayer* src = _vIncomingLayer[0];
    NNWeight* w = _vIncomingWeight[0];
    NNWeight* wsrc = w->_bShared ? w->_pSharedWeight : w;
    dsx_act_params params = {_RELUSlope, _ELUAlpha, _SELULambda};
    const uint32_t k = src->_stride;
    const void* pWeightPlanes = wsrc->SplitPlanes(w->_bTransposed, k, _localStride);
    const void* pInputPlanes = SplitInput(batch);
    dsxFatal(dsx_fc_forward_split(pInputPlanes, pWeightPlanes, w->_pbBias->_pDevData, GetIncomingUnitBuffer(), _stride, batch, k,
                                  _localStride, 0, (uint32_t)_activation, &params, pSegMax, pSegWidth),
             "NNLayer::ForwardPropagate: GEMM failure");
}

void* NNLayer::SplitInputBuffer()
{
    const size_t words = (size_t)(dsx_fc_split_bytes(_batch, _vIncomingLayer[0]->_stride) / sizeof(uint32_t));
    if (!_pbSplitInput || _pbSplitInput->_length < words) _pbSplitInput.reset(new GpuBuffer<uint32_t>(words));
    return _pbSplitInput->_pDevData;
}

const void* NNLayer::SplitInput(uint32_t batch)
{
    NNLayer* src = _vIncomingLayer[0];
    void* planes = SplitInputBuffer();
    if (_bSplitInputFresh) {   // written by the source layer's own kernel, for this batch
        _bSplitInputFresh = false;
        return planes;
    }
    dsxFatal(dsx_fc_split(src->GetUnitBuffer(), src->_stride, 0, batch, src->_stride, planes), "NNLayer::ForwardPropagate: input planes");
    return planes;
}

void NNLayer::CalculateActivation(uint32_t batch)
{
    dsx_act_params params = {_RELUSlope, _ELUAlpha, _SELULambda};
    dsxFatal(dsx_activation(GetUnitBuffer(), batch, _localStride, (uint32_t)_activation, &params), "NNLayer::CalculateActivation");
}

const string& NNLayer::GetName() const { return _name; }
const string& NNLayer::GetDataSetName() const { return _dataSet; }
NNLayer::Kind NNLayer::GetKind() const { return _kind; }
NNLayer::Type NNLayer::GetType() const { return _type; }
uint32_t NNLayer::GetAttributes() const { return _attributes; }
NNDataSetBase* NNLayer::GetDataSet() const { return _pDataSet; }
uint32_t NNLayer::GetNumDimensions() const { return _dimensions; }
tuple<uint32_t, uint32_t, uint32_t, uint32_t> NNLayer::GetDimensions() const { return std::make_tuple(_Nx, _Ny, _Nz, _Nw); }
tuple<uint32_t, uint32_t, uint32_t, uint32_t> NNLayer::GetLocalDimensions() const { return std::make_tuple(_maxX - _minX, _Ny, _Nz, _Nw); }

bool NNLayer::GetUnits(vector<NNFloat>& vUnit)
{
    if (!_pbUnit) {
        printf("NNLayer::GetUnits: Unit data not yet allocated.\n");
        return false;
    }
    if (_deferred) Materialise();
    // the whole [batch][stride] buffer comes back (the reference sizes the vector to one row only and then overruns it)
    if (vUnit.size() < _pbUnit->_length) vUnit.resize(_pbUnit->_length);
    _pbUnit->Download(vUnit.data());
    return true;
}

bool NNLayer::GetUnits(NNFloat* pUnit)
{
    if (!_pbUnit) {
        printf("NNLayer::GetUnits: Unit data not yet allocated.\n");
        return false;
    }
    if (pUnit == NULL) {
        printf("NNLayer::GetUnits: Download pointer invalid.\n");
        return false;
    }
    if (_deferred) Materialise();
    _pbUnit->Download(pUnit);
    return true;
}

bool NNLayer::SetUnits(const vector<NNFloat>& vUnit)
{
    if (!_pbUnit) {
        printf("NNLayer::SetUnits: Unit data not yet allocated.\n");
        return false;
    }
    if (vUnit.size() < _pbUnit->_length) {
        printf("NNLayer::SetUnits: Input unit data too small to set all units.\n");
        return false;
    }
    _pbUnit->Upload(vUnit.data());
    _segWidth = 0;
    _deferred = false;
    return true;
}
