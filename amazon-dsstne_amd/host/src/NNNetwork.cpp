// NNNetwork.cpp — network graph, dataset binding, PredictBatch and top-K (reference: engine/NNNetwork.cpp:404-673
// constructor, 2345-2456 propagation order, 909-988 RefreshState, 1001-1122 LoadDataSets, 1125-1158 LoadBatch, 1376-1429
// PredictBatch, 1792-1822 CalculateTopK, 1824-1988 SaveNetCDF, 3761-4057 LoadNeuralNetworkNetCDF, plus the layer and weight
// descriptor readers engine/NNLayer.cpp:3000-3337 and engine/NNWeight.cpp:90-230).
#include <algorithm>
#include <cmath>
#include <queue>

#include "NcClassic.h"
#include "amazon/dsstne/engine/NNTypes.h"

using namespace std;

std::map<NNNetwork::Kind, string> NNNetwork::_sKindMap = {{NNNetwork::Kind::FeedForward, "FeedForward"},
                                                         {NNNetwork::Kind::AutoEncoder, "AutoEncoder"}};

ostream& operator<<(ostream& out, NNNetwork::Kind& k) { return out << NNNetwork::_sKindMap[k]; }

NNNetworkDescriptor::NNNetworkDescriptor()
    : _name(""), _kind(NNNetwork::Kind::FeedForward), _errorFunction(ErrorFunction::CrossEntropy), _bShuffleIndices(true),
      _decay((NNFloat)0.0), _maxout_k(2), _LRN_k(2), _LRN_n(5), _LRN_alpha((NNFloat)0.0001), _LRN_beta((NNFloat)0.75),
      _RELUSlope((NNFloat)1.0), _ELUAlpha((NNFloat)1), _SELULambda((NNFloat)1.050701), _bSparsenessPenalty(false),
      _sparsenessPenalty_p((NNFloat)0.0), _sparsenessPenalty_beta((NNFloat)0.0), _bDenoising(false), _denoising_p((NNFloat)0.0),
      _deltaBoost_one((NNFloat)1.0), _deltaBoost_zero((NNFloat)1.0), _SMCE_oneTarget((NNFloat)0.9), _SMCE_zeroTarget((NNFloat)0.1),
      _SMCE_oneScale((NNFloat)1.0), _SMCE_zeroScale((NNFloat)1.0), _checkpoint_name("checkpoint"), _checkpoint_interval(0),
      _checkpoint_epochs(0), _bConvLayersCalculated(false)
{
}

static void fatal(const char* fmt, const char* a = "", const char* b = "")
{
    printf(fmt, a, b);
    printf("\n");
    getGpu().Shutdown();
    exit(-1);
}

NNNetwork::NNNetwork(NNNetworkDescriptor& d, uint32_t batch)
    : _name(d._name), _batch(batch), _position(0), _bExamplesFound(false), _bAllDataLoaded(true), _examples(0), _kind(d._kind),
      _errorFunction(d._errorFunction), _mode(Prediction), _bShuffleIndices(d._bShuffleIndices), _pDescriptor(NULL), _bDirty(true),
      _verbose(false), _lanes(2), _lane(0)
{
    NNDataSetBase::s_nextLane = 1;   // the first PredictBatch of a network with several lanes runs on the second one
    // keep the scalar settings (not the weight payloads) for SaveNetCDF round trips
    _pDescriptor = new NNNetworkDescriptor(d);
    _pDescriptor->_vLayerDescriptor.clear();
    _pDescriptor->_vWeightDescriptor.clear();

    for (auto& l : d._vLayerDescriptor) {
        if (_mLayer.count(l._name)) fatal("NNNetwork::NNNetwork: duplicate layer name %s.", l._name.c_str());
        if (l._type != NNLayer::Type::FullyConnected)
            fatal("NNNetwork::NNNetwork: layer %s is not fully connected; convolutional and pooling layers are not supported by this build.",
                  l._name.c_str());
        NNLayer* pLayer = new NNLayer(l, batch);
        pLayer->_lanes = _lanes;
        // layers without their own slope / alpha / lambda take the network defaults
        if (std::isnan(pLayer->_RELUSlope)) pLayer->_RELUSlope = d._RELUSlope;
        if (std::isnan(pLayer->_ELUAlpha)) pLayer->_ELUAlpha = d._ELUAlpha;
        if (std::isnan(pLayer->_SELULambda)) pLayer->_SELULambda = d._SELULambda;
        _vLayer.push_back(pLayer);
        _mLayer[pLayer->_name] = pLayer;
        if (pLayer->_kind == NNLayer::Kind::Input)
            _vInputLayer.push_back(pLayer);
        else if (pLayer->_kind == NNLayer::Kind::Output)
            _vOutputLayer.push_back(pLayer);
    }
    cout << "NNNetwork::NNNetwork: " << _vInputLayer.size() << " input layer" << (_vInputLayer.size() > 1 ? "s" : "") << endl;
    cout << "NNNetwork::NNNetwork: " << _vOutputLayer.size() << " output layer" << (_vOutputLayer.size() > 1 ? "s" : "") << endl;

    // skip connections
    for (auto l : _vLayer) {
        for (auto& s : l->_vSkip) {
            auto it = _mLayer.find(s);
            if (it == _mLayer.end()) fatal("NNNetwork::NNNetwork: unknown skip source %s for layer %s.", s.c_str(), l->_name.c_str());
            NNLayer* pLayer = it->second;
            if (pLayer->_stride != l->_stride)
                fatal("NNNetwork::NNNetwork: Layer dimensions do not match for skip connection between layer %s and %s.", l->_name.c_str(),
                      pLayer->_name.c_str());
            l->_vIncomingSkip.push_back(pLayer);
            pLayer->_vOutgoingSkip.push_back(l);
        }
    }

    // weights between layers, in descriptor order (this fixes the order of a layer's incoming sources)
    for (auto& wd : d._vWeightDescriptor) {
        auto in = _mLayer.find(wd._inputLayer), out = _mLayer.find(wd._outputLayer);
        if (in == _mLayer.end() || out == _mLayer.end())
            fatal("NNNetwork::NNNetwork: weight connects unknown layers %s and %s.", wd._inputLayer.c_str(), wd._outputLayer.c_str());
        NNWeight* pWeight = new NNWeight(*in->second, *out->second, wd._bShared, wd._bTransposed, wd._bLocked, wd._norm);
        _vWeight.push_back(pWeight);
        // a definition without values (JSON) starts from the layer's initialisation scheme; shared connections only have biases
        if (wd._vWeight.empty() || wd._vBias.empty()) pWeight->Randomize();
        if (!wd._bShared && !wd._vWeight.empty()) {
            if (wd._vWeight.size() < pWeight->_vWeight.size())
                fatal("NNNetwork::NNNetwork: too few weight values between layers %s and %s.", wd._inputLayer.c_str(), wd._outputLayer.c_str());
            std::copy(wd._vWeight.begin(), wd._vWeight.begin() + pWeight->_vWeight.size(), pWeight->_vWeight.begin());
            pWeight->_pbWeight->Upload(pWeight->_vWeight.data());
            pWeight->InvalidateSplit();
        }
        if (!wd._vBias.empty()) {
            if (wd._vBias.size() < pWeight->_vBias.size())
                fatal("NNNetwork::NNNetwork: too few bias values between layers %s and %s.", wd._inputLayer.c_str(), wd._outputLayer.c_str());
            std::copy(wd._vBias.begin(), wd._vBias.begin() + pWeight->_vBias.size(), pWeight->_vBias.begin());
            pWeight->_pbBias->Upload(pWeight->_vBias.data());
        }
    }

    // resolve shared weights in a second pass so the order of descriptors does not matter
    for (size_t i = 0; i < d._vWeightDescriptor.size(); i++) {
        NNWeightDescriptor& wd = d._vWeightDescriptor[i];
        if (!wd._bShared) continue;
        NNWeight* pWeight = _vWeight[i];
        bool bFound = false;
        for (size_t j = 0; j < _vWeight.size(); j++) {
            NNWeight* c = _vWeight[j];
            if (c->_bShared || c->_inputLayer._name != wd._sourceInputLayer || c->_outputLayer._name != wd._sourceOutputLayer) continue;
            if (wd._bTransposed) {
                if ((pWeight->_width != c->_height) || (pWeight->_height != c->_width))
                    fatal("NNNetwork::NNNetwork: Transposed dimensions for shared weights between layers %s and %s do not match",
                          pWeight->_inputLayer._name.c_str(), pWeight->_outputLayer._name.c_str());
            } else if ((pWeight->_width != c->_width) || (pWeight->_height != c->_height)) {
                fatal("NNNetwork::NNNetwork: Dimensions for shared weights between layers %s and %s do not match",
                      pWeight->_inputLayer._name.c_str(), pWeight->_outputLayer._name.c_str());
            }
            pWeight->_pSharedWeight = c;
            if (c->_sharingCount == 1) _vSharedWeight.push_back(c);
            c->_sharingCount++;
            bFound = true;
            break;
        }
        if (!bFound)
            fatal("NNNetwork::NNNetwork: Unable to locate shared weights for connection between layers %s and %s.",
                  pWeight->_inputLayer._name.c_str(), pWeight->_outputLayer._name.c_str());
    }

    CalculatePropagationOrder();
}

void NNNetwork::Randomize()
{
    for (auto pw : _vWeight) pw->Randomize();
}

NNNetwork::~NNNetwork()
{
    for (auto w : _vWeight) delete w;
    for (auto l : _vLayer) delete l;
    delete _pDescriptor;
    if (getGpu()._pNetwork == this) getGpu()._pNetwork = NULL;
    NNDataSetBase::s_nextLane = 0;
    if (dsx_is_initialized()) dsx_set_lane(0);   // whatever runs next starts on the first lane (deleting the buffers above waited for both)
}

// Forward order: every layer's priority is its longest distance from an input; a stable ordering by priority follows.
void NNNetwork::CalculatePropagationOrder()
{
    struct CompareLayer {
        bool operator()(NNLayer* l1, NNLayer* l2) { return l1->_priority < l2->_priority; }
    };
    for (auto p : _vLayer) p->_priority = (p->_kind == NNLayer::Kind::Input) ? 0 : -1;
    priority_queue<NNLayer*, vector<NNLayer*>, CompareLayer> pqueue;
    for (auto p : _vInputLayer) pqueue.push(p);
    while (!pqueue.empty()) {
        NNLayer* pLayer = pqueue.top();
        pqueue.pop();
        int32_t priority = pLayer->_priority + 1;
        for (auto p : pLayer->_vOutgoingLayer)
            if (p->_priority < priority) {
                p->_priority = priority;
                pqueue.push(p);
            }
        for (auto p : pLayer->_vOutgoingSkip)
            if (p->_priority < priority) {
                p->_priority = priority;
                pqueue.push(p);
            }
    }
    _vFPOrder.assign(_vLayer.begin(), _vLayer.end());
    stable_sort(_vFPOrder.begin(), _vFPOrder.end(), CompareLayer());
}

void NNNetwork::RefreshState()
{
    if (!_bAllDataLoaded) {
        _bAllDataLoaded = true;
        for (auto l : _vInputLayer)
            if (l->_pDataSet == NULL) {
                cout << "NNNetwork::RefreshState: Missing data set " << l->_dataSet << " for input layer " << l->_name << endl;
                _bAllDataLoaded = false;
            }
        if (_mode != Prediction)
            for (auto l : _vOutputLayer)
                if (l->_pDataSet == NULL) {
                    cout << "NNNetwork::RefreshState: Missing data set " << l->_dataSet << " for output layer " << l->_name << endl;
                    _bAllDataLoaded = false;
                }
    }
    if (_bDirty)
        for (auto l : _vLayer)
            if (l->_bDirty) l->RefreshState(this, SGD, _mode == Validation);
    if (_bDirty || (getGpu()._pNetwork != this)) getGpu().SetNeuralNetwork(this);
    _bDirty = false;
}

void NNNetwork::ClearDataSets()
{
    _examples = 0;
    _bExamplesFound = false;
    for (auto l : _vInputLayer) l->_pDataSet = NULL;
    for (auto l : _vOutputLayer) l->_pDataSet = NULL;
}

void NNNetwork::LoadDataSets(vector<NNDataSetBase*>& vData)
{
    _bAllDataLoaded = false;
    for (int pass = 0; pass < 2; pass++) {
        vector<NNLayer*>& layers = pass == 0 ? _vInputLayer : _vOutputLayer;
        const char* what = pass == 0 ? "input" : "output";
        for (auto l : layers) {
            for (auto d : vData) {
                if (l->_dataSet.compare(d->_name) != 0) continue;
                if (l->_dimensions != d->_dimensions)
                    printf("NNNetwork::LoadDataSets: Dimensionality mismatch %uD %s layer %s versus %uD data set %s\n", l->_dimensions, what,
                           l->_name.c_str(), d->_dimensions, d->_name.c_str());
                if ((l->_Nx < d->_width) || (l->_Ny < d->_height) || (l->_Nz < d->_length)) {
                    printf("NNNetwork::LoadDataSets: Data element mismatch (%u, %u, %u) %s layer %s versus (%u, %u, %u) data set %s\n", l->_Nx,
                           l->_Ny, l->_Nz, what, l->_name.c_str(), d->_width, d->_height, d->_length, d->_name.c_str());
                    break;
                }
                if (!_bExamplesFound) {
                    _examples = d->_examples;
                    _bExamplesFound = true;
                }
                if (d->_examples != _examples) {
                    printf("NNNetwork::LoadDataSets: Mismatched examples count (%u vs %u) in dataset %s\n", _examples, d->_examples,
                           d->_name.c_str());
                    break;
                }
                l->_pDataSet = d;
                if (pass == 0) l->_bSparse = d->_attributes & NNDataSetEnums::Attributes::Sparse;   // input layers take the dataset's sparseness
                l->_bDirty = true;
                printf("NNNetwork::LoadDataSets: Found data set %s for %s layer %s\n", d->_name.c_str(), what, l->_name.c_str());
                break;
            }
        }
    }
    _bDirty = true;
}

void NNNetwork::LoadBatch()
{
    if (_bDirty) RefreshState();
    uint32_t batch = _batch;
    if (_position + batch > _examples) batch = _examples - _position;
    for (auto l : _vInputLayer) l->LoadPredictionBatch(_position, batch);
}

void NNNetwork::PredictBatch(uint32_t layers)
{
    if (layers > _vLayer.size()) {
        printf("NNNetwork::PredictBatch: Attempt to predict more layers than present in neural network %s\n", _name.c_str());
        return;
    }
    if (_mode != Prediction) {
        _mode = Prediction;
        _bDirty = true;
    }
    if (_bDirty) {
        RefreshState();
        if (!_bAllDataLoaded) {
            cout << "NNNetwork::PredictBatch: Attempt to predict with neural network " << _name << " without providing data sets" << endl;
            cout << "for all input and output layers." << endl;
            getGpu().Shutdown();
            exit(-1);
        }
    }
    if (_lanes > 1) {
        // this batch takes the lane that has been idle longest
        _lane = (_lane + 1) % _lanes;
        for (auto l : _vLayer) l->SwitchLane(_lane);
        dsxFatal(dsx_set_lane((int)_lane), "NNNetwork::PredictBatch: lane");
    }
    NNDataSetBase::s_nextLane = (int)((_lane + 1) % _lanes);   // where a LoadSparseData for the next batch should go
    uint32_t batch = _batch;
    if (_position + batch > _examples) batch = _examples - _position;
    ClearUpdates();
    LoadBatch();
    for (auto l : _vLayer) l->_bSplitInputFresh = false;   // planes a layer wrote for its consumer belong to the batch they were written in
    for (auto l : _vFPOrder) l->ForwardPropagate(_position, batch, false);
}

bool NNNetwork::SetLanes(uint32_t lanes)
{
    if (lanes < 1 || lanes > DSX_MAX_LANES) {
        printf("NNNetwork::SetLanes: %u lanes requested (1..%d).\n", lanes, DSX_MAX_LANES);
        return false;
    }
    if (lanes == _lanes) return true;
    dsxFatal(dsx_sync(), "NNNetwork::SetLanes");
    _lanes = lanes;
    _lane = 0;
    dsxFatal(dsx_set_lane(0), "NNNetwork::SetLanes");
    NNDataSetBase::s_nextLane = (lanes > 1) ? 1 : 0;
    for (auto l : _vLayer) {
        l->_lanes = lanes;
        l->_currentLane = 0;
        l->_bDirty = true;   // unit buffers are allocated anew
    }
    _bDirty = true;
    return true;
}

// The deferred output layer and its top-K in one call; the layer's result is not stored.
void NNNetwork::LayerWithTopK(NNLayer* pLayer, uint32_t k, uint32_t batch, const uint32_t* pIndex, const uint64_t* pFilterStart,
                              const uint64_t* pFilterEnd, const uint32_t* pFilterIndex, NNFloat* pKey, uint32_t* pValue)
{
    NNLayer* src = pLayer->_vIncomingLayer[0];
    NNWeight* w = pLayer->_vIncomingWeight[0];
    NNWeight* wsrc = w->_bShared ? w->_pSharedWeight : w;
    dsx_act_params params = {pLayer->_RELUSlope, pLayer->_ELUAlpha, pLayer->_SELULambda};
    if (pLayer->UseSplitProducts(batch)) {
        const void* pInputPlanes = pLayer->SplitInput(batch);
        dsxFatal(dsx_fc_topk_split(src->GetUnitBuffer(), src->_stride, wsrc->_pbWeight->_pDevData, pInputPlanes,
                                   wsrc->SplitPlanes(false, src->_stride, pLayer->_localStride), w->_pbBias->_pDevData, batch, src->_stride,
                                   pLayer->_localStride, (uint32_t)pLayer->_activation, &params, k, pKey, pValue, _position, pIndex,
                                   pFilterStart, pFilterEnd, pFilterIndex),
                 "NNNetwork::CalculateTopK: output layer with top-K");
        return;
    }
    dsxFatal(dsx_fc_topk(src->GetUnitBuffer(), src->_stride, wsrc->_pbWeight->_pDevData, w->_pbBias->_pDevData, batch, src->_stride,
                         pLayer->_localStride, (uint32_t)pLayer->_activation, &params, k, pKey, pValue, _position, pIndex, pFilterStart,
                         pFilterEnd, pFilterIndex),
             "NNNetwork::CalculateTopK: output layer with top-K");
}

bool NNNetwork::SetSplitProducts(bool bSplit)
{
    dsx_device_info info;
    dsxFatal(dsx_get_device_info(&info), "NNNetwork::SetSplitProducts");
    for (auto l : _vLayer) {
        l->_bSplitProducts = bSplit;
        l->_splitMinTiles = 2u * info.compute_units;
    }
    // (also the way to say that weights were written through NNWeight::GetWeightBuffer: the planes are built again on next use)
    for (auto w : _vWeight) {
        w->InvalidateSplit();
        if (!bSplit) {
            w->_pbSplit[0].reset();
            w->_pbSplit[1].reset();
        }
    }
    return true;
}

bool NNNetwork::SetDeferredOutput(bool bDefer)
{
    for (auto l : _vLayer) {
        if (!bDefer && l->_deferred) l->Materialise();
        l->_bDeferOutput = bDefer;
    }
    return true;
}

void NNNetwork::CalculateTopK(const string& layer, uint32_t k, GpuBuffer<NNFloat>* pbKey, GpuBuffer<uint32_t>* pbValue)
{
    auto it = _mLayer.find(layer);
    if (it == _mLayer.end()) {
        printf("NNNetwork::CalculateTopK: Unknown layer %s.\n", layer.c_str());
        return;
    }
    NNLayer* pLayer = it->second;
    if (k > 128) {
        printf("NNNetwork::CalculateTopK: Can only calculate 128 or fewer elements.\n");
        return;
    }
    if (k > pLayer->_Nx * pLayer->_Ny * pLayer->_Nz) {
        printf("NNNetwork::CalculateTopK: Layer has fewer elements than k (%u vs %u).\n", k, pLayer->_Nx * pLayer->_Ny * pLayer->_Nz);
        return;
    }
    if (!pLayer->_pbUnit) {
        printf("NNNetwork::CalculateTopK: Layer %s has no unit buffer.\n", layer.c_str());
        return;
    }
    uint32_t batch = _batch;
    if (_position + batch > _examples) batch = _examples - _position;
    if (pLayer->_deferred)
        LayerWithTopK(pLayer, k, batch, NULL, NULL, NULL, NULL, pbKey->_pDevData, pbValue->_pDevData);
    else if (pLayer->_segWidth != 0 && pLayer->_pbSegMax)
        dsxFatal(dsx_topk_guided(pLayer->_pbUnit->_pDevData, pbKey->_pDevData, pbValue->_pDevData, batch, pLayer->_localStride, k,
                                 pLayer->_pbSegMax->_pDevData, pLayer->_segWidth, 0, NULL, NULL, NULL, NULL, NULL),
                 "NNNetwork::CalculateTopK");
    else
        kCalculateTopK(pLayer->_pbUnit->_pDevData, pbKey->_pDevData, pbValue->_pDevData, batch, pLayer->_localStride, k);
}

void NNNetwork::CalculateFilteredTopK(const string& layer, uint32_t k, NNDataSetBase* pFilter, GpuBuffer<NNFloat>* pbKey,
                                      GpuBuffer<uint32_t>* pbValue, bool bUseValues)
{
    auto it = _mLayer.find(layer);
    if (it == _mLayer.end()) {
        printf("NNNetwork::CalculateFilteredTopK: Unknown layer %s.\n", layer.c_str());
        return;
    }
    NNLayer* pLayer = it->second;
    if (k > 256) {
        printf("NNNetwork::CalculateFilteredTopK: Can only calculate 256 or fewer elements.\n");
        return;
    }
    if (k > pLayer->_Nx * pLayer->_Ny * pLayer->_Nz) {
        printf("NNNetwork::CalculateFilteredTopK: Layer has fewer elements than k (%u vs %u).\n", k, pLayer->_Nx * pLayer->_Ny * pLayer->_Nz);
        return;
    }
    if (!pLayer->_pbUnit || !pFilter || !(pFilter->_attributes & NNDataSetEnums::Sparse) || !pFilter->_pbSparseStart) {
        printf("NNNetwork::CalculateFilteredTopK: Layer %s has no unit buffer or the filter is not a sparse dataset.\n", layer.c_str());
        return;
    }
    uint32_t batch = _batch;
    if (_position + batch > _examples) batch = _examples - _position;
    // Listed items are multiplied by 0 unless the caller asks for the dataset's own (float) values as multipliers.
    const NNFloat* pMul = NULL;
    if (bUseValues && !(pFilter->_attributes & NNDataSetEnums::Boolean) && pFilter->_dataType == NNDataSetEnums::Float) {
        NNDataSet<float>* pf = dynamic_cast<NNDataSet<float>*>(pFilter);
        if (pf && pf->_pbSparseData) pMul = pf->_pbSparseData->_pDevData;
    }
    pFilter->NoteSparseRead();
    const uint32_t* pIndex = (pFilter->_attributes & NNDataSetEnums::Indexed) ? pFilter->_pbIndex->_pDevData : NULL;
    if (pLayer->_deferred) {
        if (pMul == NULL) {
            LayerWithTopK(pLayer, k, batch, pIndex, pFilter->_pbSparseStart->_pDevData, pFilter->_pbSparseEnd->_pDevData,
                          pFilter->_pbSparseIndex->_pDevData, pbKey->_pDevData, pbValue->_pDevData);
            return;
        }
        pLayer->Materialise();   // multipliers other than 0 need the listed items' scores
    }
    // with segment maxima of the current batch (left by the layer's dense kernel) only the segments that can hold a result are read
    const NNFloat* pSegMax = (pLayer->_segWidth != 0 && pLayer->_pbSegMax) ? pLayer->_pbSegMax->_pDevData : NULL;
    dsxFatal(dsx_topk_guided(pLayer->_pbUnit->_pDevData, pbKey->_pDevData, pbValue->_pDevData, batch, pLayer->_localStride, k, pSegMax,
                             pLayer->_segWidth, _position, pIndex, pFilter->_pbSparseStart->_pDevData, pFilter->_pbSparseEnd->_pDevData,
                             pFilter->_pbSparseIndex->_pDevData, pMul),
             "NNNetwork::CalculateFilteredTopK");
}

void NNNetwork::CalculateFilteredTopK(const string& layer, uint32_t k, const uint64_t* pFilterStart, const uint64_t* pFilterEnd,
                                      const uint32_t* pFilterIndex, const NNFloat* pFilterMul, NNFloat* pKey, uint32_t* pValue)
{
    auto it = _mLayer.find(layer);
    if (it == _mLayer.end() || !it->second->_pbUnit) {
        printf("NNNetwork::CalculateFilteredTopK: Unknown layer %s or no unit buffer.\n", layer.c_str());
        return;
    }
    NNLayer* pLayer = it->second;
    if (k > 256 || k > pLayer->_Nx * pLayer->_Ny * pLayer->_Nz) {
        printf("NNNetwork::CalculateFilteredTopK: k = %u does not fit layer %s (256 at most).\n", k, layer.c_str());
        return;
    }
    uint32_t batch = _batch;
    if (_position + batch > _examples) batch = _examples - _position;
    if (pLayer->_deferred) {
        if (pFilterMul == NULL) {
            LayerWithTopK(pLayer, k, batch, NULL, pFilterStart, pFilterEnd, pFilterIndex, pKey, pValue);
            return;
        }
        pLayer->Materialise();
    }
    const NNFloat* pSegMax = (pLayer->_segWidth != 0 && pLayer->_pbSegMax) ? pLayer->_pbSegMax->_pDevData : NULL;
    dsxFatal(dsx_topk_guided(pLayer->_pbUnit->_pDevData, pKey, pValue, batch, pLayer->_localStride, k, pSegMax, pLayer->_segWidth, _position,
                             NULL, pFilterStart, pFilterEnd, pFilterIndex, pFilterMul),
             "NNNetwork::CalculateFilteredTopK");
}

void NNNetwork::SetBatch(uint32_t batch)
{
    if (batch != _batch) {
        _batch = batch;
        for (auto pL : _vLayer) pL->SetBatch(batch);
        _bDirty = true;
        printf("NNNetwork::SetBatch: Batch size set to %d.\n", _batch);
    }
}

void NNNetwork::SetPosition(uint32_t position)
{
    if (_bExamplesFound) {
        if (position < _examples)
            _position = position;
        else
            printf("NNNetwork::SetPosition: Invalid position setting: %u, maximum %u\n", position, _examples);
    } else {
        printf("NNNetwork::SetPosition: Illegal attempt to set position without examples count information.\n");
    }
}

void NNNetwork::SetShuffleIndices(bool bShuffleIndices)
{
    // index shuffling only acts in training mode (engine/GpuTypes.cpp:495); the flag is kept for file round trips
    _bShuffleIndices = bShuffleIndices;
    printf("NNNetwork::SetShuffleIndices: Index shuffling is now %s\n", (_bShuffleIndices ? "on" : "off"));
}

void NNNetwork::SetCPUValidate(bool bValidate) { getGpu().SetCPUValidate(bValidate); }

unsigned int NNNetwork::GetBatch() const { return _batch; }
uint32_t NNNetwork::GetExamples() const { return _examples; }
uint32_t NNNetwork::GetPosition() const { return _position; }
const string& NNNetwork::GetName() const { return _name; }

NNLayer* NNNetwork::GetLayer(const string& layer) const
{
    auto itr = _mLayer.find(layer);
    if (itr == _mLayer.end()) {
        printf("NNNetwork::GetLayerDimensions: Unknown layer %s.\n", layer.c_str());
        return NULL;
    }
    return itr->second;
}

vector<string> NNNetwork::GetLayers() const
{
    vector<string> v;
    for (auto l : _vLayer) v.push_back(l->_name);
    return v;
}

vector<const NNLayer*>::iterator NNNetwork::GetLayers(NNLayer::Kind layerKind, vector<const NNLayer*>& layers) const
{
    int count = 0;
    for (auto l : _vLayer)
        if (l->_kind == layerKind) {
            layers.insert(layers.end(), l);
            ++count;
        }
    return layers.end() - count;
}

NNFloat* NNNetwork::GetUnitBuffer(const string& layer)
{
    auto itr = _mLayer.find(layer);
    if (itr == _mLayer.end()) {
        printf("NNNetwork::GetUnitBuffer: Unknown layer %s.\n", layer.c_str());
        return NULL;
    }
    if (itr->second->_deferred) itr->second->Materialise();
    // the caller gets a writable device pointer: the segment maxima of the batch may not describe the units any longer
    itr->second->_segWidth = 0;
    // The reference's callers follow this call with a plain cudaMemcpy or a kernel of their own
    // (utils/NNRecsGenerator.cpp:83, java/src/main/native/com_amazon_dsstne_Dsstne.cpp:366), which the default stream ordered
    // after the forward pass.  The lanes' streams are not ordered against the null stream, so the batch that filled this
    // buffer is waited for here; a batch in flight on another lane keeps running.
    dsxFatal(dsx_sync_lane((int)_lane), "NNNetwork::GetUnitBuffer");
    return itr->second->GetUnitBuffer();
}

uint64_t NNNetwork::GetBufferSize(const string& layer) const
{
    auto itr = _mLayer.find(layer);
    if (itr == _mLayer.end()) {
        printf("NNNetwork::GetDeltaBuffer: Unknown layer %s.\n", layer.c_str());
        return 0;
    }
    return itr->second->GetBufferSize();
}

NNWeight* NNNetwork::GetWeight(const string& inputLayer, const string& outputLayer) const
{
    auto in = _mLayer.find(inputLayer);
    if (in == _mLayer.end()) {
        printf("NNNetwork::GetWeight: Unknown input layer %s.\n", inputLayer.c_str());
        return NULL;
    }
    auto out = _mLayer.find(outputLayer);
    if (out == _mLayer.end()) {
        printf("NNNetwork::GetWeight: Unknown output layer %s.\n", outputLayer.c_str());
        return NULL;
    }
    for (auto p : _vWeight)
        if ((&(p->_inputLayer) == in->second) && (&(p->_outputLayer) == out->second)) return p;
    printf("NNNetwork::GetWeight: No set of weights connecting layer %s to layer %s.\n", inputLayer.c_str(), outputLayer.c_str());
    return NULL;
}

NNFloat* NNNetwork::GetWeightBuffer(const string& inputLayer, const string& outputLayer)
{
    NNWeight* w = GetWeight(inputLayer, outputLayer);
    return w ? w->GetWeightBuffer() : NULL;
}

// ---------------------------------------------------------------------------------------------------------------- file I/O

static float attF(const ncc::Reader& nc, const string& name, float dflt)
{
    return nc.hasAtt(name) ? (float)nc.att(name).asDouble() : dflt;
}
static uint32_t attU(const ncc::Reader& nc, const string& name, uint32_t dflt)
{
    return nc.hasAtt(name) ? (uint32_t)nc.att(name).asUInt64() : dflt;
}

bool LoadNNNetworkDescriptorNetCDF(const string& fname, NNNetworkDescriptor& nd)
{
    try {
        ncc::Reader nc(fname);
        nc.att("version");   // must be present (engine/NNNetwork.cpp:3789-3794)
        nd._name = nc.att("name").asString();
        nd._kind = (NNNetwork::Kind)nc.att("kind").asUInt64();
        nd._errorFunction = (ErrorFunction)nc.att("errorFunction").asUInt64();
        nd._decay = attF(nc, "decay", 0.0f);
        nd._maxout_k = attU(nc, "maxout_k", 2);
        nd._LRN_k = attF(nc, "LRN_k", 2.0f);
        nd._LRN_n = attU(nc, "LRN_n", 5);
        nd._LRN_alpha = attF(nc, "LRN_alpha", 0.0001f);
        nd._LRN_beta = attF(nc, "LRN_beta", 0.75f);
        nd._bSparsenessPenalty = attU(nc, "bSparsenessPenalty", 0) != 0;
        nd._sparsenessPenalty_p = attF(nc, "sparsenessPenalty_p", 0.0f);
        nd._sparsenessPenalty_beta = attF(nc, "sparsenessPenalty_beta", 0.0f);
        nd._bDenoising = attU(nc, "bDenoising", 0) != 0;
        nd._denoising_p = attF(nc, "denoising_p", 0.0f);
        nd._deltaBoost_one = attF(nc, "deltaBoost_one", 1.0f);
        nd._deltaBoost_zero = attF(nc, "deltaBoost_zero", 1.0f);
        nd._SMCE_oneScale = attF(nc, "SMCE_oneScale", 1.0f);
        nd._SMCE_zeroScale = attF(nc, "SMCE_zeroScale", 1.0f);
        nd._SMCE_oneTarget = attF(nc, "SMCE_oneTarget", 0.9f);
        nd._SMCE_zeroTarget = attF(nc, "SMCE_zeroTarget", 0.1f);
        nd._bShuffleIndices = attU(nc, "ShuffleIndices", 1) != 0;
        if (nc.hasAtt("checkpoint_name")) nd._checkpoint_name = nc.att("checkpoint_name").asString();
        nd._checkpoint_interval = (int32_t)attU(nc, "checkpoint_interval", 0);
        nd._checkpoint_epochs = (int32_t)attU(nc, "checkpoint_epochs", 0);
        nd._bConvLayersCalculated = true;

        const uint32_t layers = (uint32_t)nc.att("layers").asUInt64();
        for (uint32_t i = 0; i < layers; i++) {
            const string p = "layer" + std::to_string(i) + "_";
            NNLayerDescriptor ld;
            ld._name = nc.att(p + "name").asString();
            ld._kind = (NNLayer::Kind)nc.att(p + "kind").asUInt64();
            ld._type = (NNLayer::Type)nc.att(p + "type").asUInt64();
            ld._poolingFunction = (PoolingFunction)attU(nc, p + "poolingfunction", 0);
            ld._dataSet = nc.att(p + "dataSet").asString();
            ld._Nx = (uint32_t)nc.att(p + "Nx").asUInt64();
            ld._Ny = (uint32_t)nc.att(p + "Ny").asUInt64();
            ld._Nz = (uint32_t)nc.att(p + "Nz").asUInt64();
            ld._Nw = (uint32_t)nc.att(p + "Nw").asUInt64();
            ld._dimensions = (uint32_t)nc.att(p + "dimensions").asUInt64();
            ld._kernelX = attU(nc, p + "kernelX", 1);
            ld._kernelY = attU(nc, p + "kernelY", 1);
            ld._kernelZ = attU(nc, p + "kernelZ", 1);
            ld._kernelDimensions = attU(nc, p + "kernelDimensions", 1);
            ld._kernelStrideX = attU(nc, p + "kernelStrideX", 1);
            ld._kernelStrideY = attU(nc, p + "kernelStrideY", 1);
            ld._kernelStrideZ = attU(nc, p + "kernelStrideZ", 1);
            ld._kernelPaddingX = attU(nc, p + "kernelPaddingX", 0);
            ld._kernelPaddingY = attU(nc, p + "kernelPaddingY", 0);
            ld._kernelPaddingZ = attU(nc, p + "kernelPaddingZ", 0);
            ld._pDropout = attF(nc, p + "pDropout", 0.0f);
            ld._weightInit = (WeightInitialization)attU(nc, p + "weightInit", 0);
            ld._weightInitScale = attF(nc, p + "weightInitScale", 1.0f);
            ld._biasInit = attF(nc, p + "biasInit", 0.0f);
            ld._weightNorm = attF(nc, p + "weightNorm", 0.0f);
            ld._deltaNorm = attF(nc, p + "deltaNorm", 0.0f);
            ld._activation = (Activation)nc.att(p + "activation").asUInt64();
            ld._sparsenessPenalty_p = attF(nc, p + "sparsenessPenalty_p", 0.0f);
            ld._sparsenessPenalty_beta = attF(nc, p + "sparsenessPenalty_beta", 0.0f);
            ld._RELUSlope = attF(nc, p + "RELUSlope", NAN);
            ld._ELUAlpha = attF(nc, p + "ELUAlpha", NAN);
            ld._SELULambda = attF(nc, p + "SELULambda", NAN);
            ld._attributes = (uint32_t)nc.att(p + "attributes").asUInt64();
            const uint32_t sources = attU(nc, p + "sources", 0);
            for (uint32_t j = 0; j < sources; j++) ld._vSource.push_back(nc.att(p + "source" + std::to_string(j)).asString());
            const uint32_t skips = attU(nc, p + "skips", 0);
            for (uint32_t j = 0; j < skips; j++) ld._vSkip.push_back(nc.att(p + "skip" + std::to_string(j)).asString());
            nd._vLayerDescriptor.push_back(ld);
        }

        const uint32_t weights = (uint32_t)nc.att("weights").asUInt64();
        for (uint32_t i = 0; i < weights; i++) {
            const string p = "weight" + std::to_string(i) + "_";
            NNWeightDescriptor wd;
            wd._inputLayer = nc.att(p + "inputLayer").asString();
            wd._outputLayer = nc.att(p + "outputLayer").asString();
            wd._norm = attF(nc, p + "norm", 0.0f);
            wd._bShared = nc.att(p + "bShared").asUInt64() != 0;
            if (wd._bShared) {
                wd._sourceInputLayer = nc.att(p + "sourceInputLayer").asString();
                wd._sourceOutputLayer = nc.att(p + "sourceOutputLayer").asString();
                wd._bTransposed = nc.att(p + "bTransposed").asUInt64() != 0;
            }
            wd._bLocked = attU(nc, p + "bLocked", 0) != 0;
            wd._width = nc.att(p + "width").asUInt64();
            wd._height = nc.att(p + "height").asUInt64();
            wd._length = nc.att(p + "length").asUInt64();
            wd._depth = nc.hasAtt(p + "depth") ? nc.att(p + "depth").asUInt64() : 1;
            wd._breadth = nc.hasAtt(p + "breadth") ? nc.att(p + "breadth").asUInt64() : 1;
            nc.read<NNFloat>(p + "bias", wd._vBias);
            if (!wd._bShared) nc.read<NNFloat>(p + "weights", wd._vWeight);
            nd._vWeightDescriptor.push_back(std::move(wd));
        }
    } catch (std::exception& e) {
        cout << "Exception: " << e.what() << endl;
        return false;
    }
    return true;
}

static void writeDescriptor(ncc::Writer& nc, const NNNetworkDescriptor& nd)
{
    nc.putAttFloat("version", NN_VERSION);
    nc.putAttString("name", nd._name);
    nc.putAttUInt("kind", nd._kind);
    nc.putAttUInt("errorFunction", nd._errorFunction);
    nc.putAttInt("maxout_k", (int32_t)nd._maxout_k);
    nc.putAttFloat("decay", nd._decay);
    nc.putAttFloat("LRN_k", nd._LRN_k);
    nc.putAttInt("LRN_n", (int32_t)nd._LRN_n);
    nc.putAttFloat("LRN_alpha", nd._LRN_alpha);
    nc.putAttFloat("LRN_beta", nd._LRN_beta);
    nc.putAttUInt("bSparsenessPenalty", nd._bSparsenessPenalty);
    nc.putAttFloat("sparsenessPenalty_p", nd._sparsenessPenalty_p);
    nc.putAttFloat("sparsenessPenalty_beta", nd._sparsenessPenalty_beta);
    nc.putAttUInt("bDenoising", nd._bDenoising);
    nc.putAttFloat("denoising_p", nd._denoising_p);
    nc.putAttFloat("deltaBoost_one", nd._deltaBoost_one);
    nc.putAttFloat("deltaBoost_zero", nd._deltaBoost_zero);
    nc.putAttFloat("SMCE_oneScale", nd._SMCE_oneScale);
    nc.putAttFloat("SMCE_zeroScale", nd._SMCE_zeroScale);
    nc.putAttFloat("SMCE_oneTarget", nd._SMCE_oneTarget);
    nc.putAttFloat("SMCE_zeroTarget", nd._SMCE_zeroTarget);
    nc.putAttUInt("ShuffleIndices", nd._bShuffleIndices);
    nc.putAttString("checkpoint_name", nd._checkpoint_name);
    nc.putAttInt("checkpoint_interval", nd._checkpoint_interval);
    nc.putAttInt("checkpoint_epochs", nd._checkpoint_epochs);
    nc.putAttUInt("layers", (uint32_t)nd._vLayerDescriptor.size());
    for (size_t i = 0; i < nd._vLayerDescriptor.size(); i++) {
        const NNLayerDescriptor& l = nd._vLayerDescriptor[i];
        const string p = "layer" + std::to_string(i) + "_";
        nc.putAttString(p + "name", l._name);
        nc.putAttUInt(p + "kind", l._kind);
        nc.putAttUInt(p + "type", l._type);
        nc.putAttUInt(p + "poolingfunction", l._poolingFunction);
        nc.putAttString(p + "dataSet", l._dataSet);
        nc.putAttUInt(p + "Nx", l._Nx);
        nc.putAttUInt(p + "Ny", l._Ny);
        nc.putAttUInt(p + "Nz", l._Nz);
        nc.putAttUInt(p + "Nw", l._Nw);
        nc.putAttUInt(p + "dimensions", l._dimensions);
        nc.putAttUInt(p + "kernelX", l._kernelX);
        nc.putAttUInt(p + "kernelY", l._kernelY);
        nc.putAttUInt(p + "kernelZ", l._kernelZ);
        nc.putAttUInt(p + "kernelDimensions", l._kernelDimensions);
        nc.putAttUInt(p + "kernelStrideX", l._kernelStrideX);
        nc.putAttUInt(p + "kernelStrideY", l._kernelStrideY);
        nc.putAttUInt(p + "kernelStrideZ", l._kernelStrideZ);
        nc.putAttUInt(p + "kernelPaddingX", l._kernelPaddingX);
        nc.putAttUInt(p + "kernelPaddingY", l._kernelPaddingY);
        nc.putAttUInt(p + "kernelPaddingZ", l._kernelPaddingZ);
        nc.putAttFloat(p + "pDropout", l._pDropout);
        nc.putAttUInt(p + "weightInit", l._weightInit);
        nc.putAttFloat(p + "weightInitScale", l._weightInitScale);
        nc.putAttFloat(p + "biasInit", l._biasInit);
        nc.putAttFloat(p + "weightNorm", l._weightNorm);
        nc.putAttFloat(p + "deltaNorm", l._deltaNorm);
        nc.putAttUInt(p + "activation", l._activation);
        nc.putAttFloat(p + "sparsenessPenalty_p", l._sparsenessPenalty_p);
        nc.putAttFloat(p + "sparsenessPenalty_beta", l._sparsenessPenalty_beta);
        nc.putAttFloat(p + "RELUSlope", l._RELUSlope);
        nc.putAttFloat(p + "ELUAlpha", l._ELUAlpha);
        nc.putAttFloat(p + "SELULambda", l._SELULambda);
        nc.putAttUInt(p + "attributes", l._attributes);
        nc.putAttUInt(p + "sources", (uint32_t)l._vSource.size());
        for (size_t j = 0; j < l._vSource.size(); j++) nc.putAttString(p + "source" + std::to_string(j), l._vSource[j]);
        nc.putAttUInt(p + "skips", (uint32_t)l._vSkip.size());
        for (size_t j = 0; j < l._vSkip.size(); j++) nc.putAttString(p + "skip" + std::to_string(j), l._vSkip[j]);
    }
    nc.putAttUInt("weights", (uint32_t)nd._vWeightDescriptor.size());
    for (size_t i = 0; i < nd._vWeightDescriptor.size(); i++) {
        const NNWeightDescriptor& w = nd._vWeightDescriptor[i];
        const string p = "weight" + std::to_string(i) + "_";
        nc.putAttString(p + "inputLayer", w._inputLayer);
        nc.putAttString(p + "outputLayer", w._outputLayer);
        nc.putAttUInt64(p + "width", w._width);
        nc.putAttUInt64(p + "height", w._height);
        nc.putAttUInt64(p + "length", w._length);
        nc.putAttUInt64(p + "depth", w._depth);
        nc.putAttUInt64(p + "breadth", w._breadth);
        nc.putAttUInt(p + "bShared", w._bShared);
        nc.putAttUInt(p + "bLocked", w._bLocked);
        nc.putAttFloat(p + "norm", w._norm);
        const uint32_t biasDim = nc.addDim(p + "biasDim", w._vBias.size());
        nc.addVar(p + "bias", ncc::NC_FLOAT, biasDim, w._vBias.data());
        if (w._bShared) {
            nc.putAttUInt(p + "bTransposed", w._bTransposed);
            nc.putAttString(p + "sourceInputLayer", w._sourceInputLayer);
            nc.putAttString(p + "sourceOutputLayer", w._sourceOutputLayer);
        } else {
            const uint32_t weightDim = nc.addDim(p + "weightDim", w._vWeight.size());
            nc.addVar(p + "weights", ncc::NC_FLOAT, weightDim, w._vWeight.data());
        }
    }
}

bool SaveNNNetworkDescriptorNetCDF(const string& fname, const NNNetworkDescriptor& nd)
{
    try {
        ncc::Writer nc;
        writeDescriptor(nc, nd);
        nc.write(fname);
    } catch (std::exception& e) {
        cout << "Exception: " << e.what() << endl;
        return false;
    }
    return true;
}

bool NNNetwork::SaveNetCDF(const string& fname)
{
    // Rebuild a full descriptor from the live network (weights are downloaded from the device).
    NNNetworkDescriptor nd(*_pDescriptor);
    nd._name = _name;
    nd._bShuffleIndices = _bShuffleIndices;
    for (auto l : _vLayer) {
        NNLayerDescriptor ld;
        ld._name = l->_name;
        ld._kind = l->_kind;
        ld._type = l->_type;
        ld._dataSet = l->_dataSet;
        ld._vSource = l->_vSource;
        ld._vSkip = l->_vSkip;
        ld._Nx = l->_Nx;
        ld._Ny = l->_Ny;
        ld._Nz = l->_Nz;
        ld._Nw = l->_Nw;
        ld._dimensions = l->_dimensions;
        ld._pDropout = l->_pDropout;
        ld._activation = l->_activation;
        ld._RELUSlope = l->_RELUSlope;
        ld._ELUAlpha = l->_ELUAlpha;
        ld._SELULambda = l->_SELULambda;
        ld._attributes = l->_bSparse ? NNLayer::Attributes::Sparse : NNLayer::Attributes::None;
        nd._vLayerDescriptor.push_back(ld);
    }
    for (auto w : _vWeight) {
        NNWeightDescriptor wd;
        wd._inputLayer = w->_inputLayer._name;
        wd._outputLayer = w->_outputLayer._name;
        wd._width = w->_width;
        wd._height = w->_height;
        wd._length = w->_length;
        wd._depth = w->_depth;
        wd._breadth = w->_breadth;
        wd._bShared = w->_bShared;
        wd._bTransposed = w->_bTransposed;
        wd._bLocked = w->_bLocked;
        wd._norm = w->_norm;
        w->GetBiases(wd._vBias);
        if (w->_bShared) {
            wd._sourceInputLayer = w->_pSharedWeight->_inputLayer._name;
            wd._sourceOutputLayer = w->_pSharedWeight->_outputLayer._name;
        } else {
            w->GetWeights(wd._vWeight);
        }
        nd._vWeightDescriptor.push_back(std::move(wd));
    }
    if (!SaveNNNetworkDescriptorNetCDF(fname, nd)) {
        printf("NNNetwork::SaveNetCDF Error opening binary output file %s to save neural network %s.\n", fname.c_str(), _name.c_str());
        getGpu().Shutdown();
        exit(-1);
    }
    return true;
}

bool SaveNeuralNetworkNetCDF(const NNNetwork& net, const string& fname) { return const_cast<NNNetwork&>(net).SaveNetCDF(fname); }

NNNetwork* CreateNeuralNetwork(NNNetworkDescriptor& d, const uint32_t batch)
{
    NNNetwork* pNetwork = new NNNetwork(d, batch);
    pNetwork->RefreshState();
    return pNetwork;
}

NNNetwork* LoadNeuralNetworkNetCDF(const string& fname, const uint32_t batch)
{
    NNNetworkDescriptor nd;
    if (!LoadNNNetworkDescriptorNetCDF(fname, nd)) {
        cout << "Exception: NNetWork::NNetwork: Error reading NetCDF input file " << fname << endl;
        getGpu().Shutdown();
        exit(-1);
    }
    return CreateNeuralNetwork(nd, batch);
}
