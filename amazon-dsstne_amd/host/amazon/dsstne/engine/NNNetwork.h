// NNNetwork.h — the network object of the inference path (public surface of the reference's engine/NNNetwork.h).
// Graph of fully connected layers, dataset binding, batch position, PredictBatch and top-K.  Training, checkpoints and
// multi-process buffers are not part of this build.
#ifndef DSSTNE_AMD_NNNETWORK_H
#define DSSTNE_AMD_NNNETWORK_H

#include "GpuTypes.h"
#include "NNDefs.h"
#include "NNLayer.h"
#include "NNWeight.h"

struct NNNetworkDescriptor;
struct NNDataSetBase;

class NNNetwork {
public:
    friend class NNLayer;
    friend class NNWeight;
    enum Kind { FeedForward, AutoEncoder };
    static std::map<Kind, string> _sKindMap;

private:
    friend NNNetwork* LoadNeuralNetworkNetCDF(const string& fname, const uint32_t batch);
    friend NNNetwork* CreateNeuralNetwork(NNNetworkDescriptor& d, const uint32_t batch);
    friend bool SaveNeuralNetworkNetCDF(const NNNetwork& net, const string& fname);

    string _name;
    uint32_t _batch;
    uint32_t _position;
    bool _bExamplesFound;
    bool _bAllDataLoaded;
    uint32_t _examples;
    const Kind _kind;
    ErrorFunction _errorFunction;
    Mode _mode;
    bool _bShuffleIndices;
    NNNetworkDescriptor* _pDescriptor;          // scalar settings kept for SaveNetCDF round trips
    vector<NNLayer*> _vLayer;
    vector<NNLayer*> _vInputLayer;
    vector<NNLayer*> _vOutputLayer;
    vector<NNWeight*> _vWeight;
    vector<NNWeight*> _vSharedWeight;
    vector<NNDataSetBase*> _vData;
    vector<NNLayer*> _vFPOrder;
    map<string, NNLayer*> _mLayer;
    bool _bDirty;
    bool _verbose;
    uint32_t _lanes;                            // 1: one set of unit buffers, one stream; 2 (default) to DSX_MAX_LANES: consecutive batches take turns
    uint32_t _lane;                             // the lane of the current batch

    NNNetwork(NNNetworkDescriptor& nd, uint32_t batch = DefaultBatch);
    void CalculatePropagationOrder();
    void LoadBatch();
    void RefreshState();
    void ClearUpdates() {}
    void LayerWithTopK(NNLayer* pLayer, uint32_t k, uint32_t batch, const uint32_t* pIndex, const uint64_t* pFilterStart,
                       const uint64_t* pFilterEnd, const uint32_t* pFilterIndex, NNFloat* pKey, uint32_t* pValue);

public:
    ~NNNetwork();
    void ClearDataSets();
    void LoadDataSets(vector<NNDataSetBase*>& vData);
    void PredictBatch(uint32_t layers = 0);
    void CalculateTopK(const string& layer, uint32_t k, GpuBuffer<NNFloat>* pbKey, GpuBuffer<uint32_t>* pbValue);
    // Filtered recommendations in one device pass: the top-k of `layer` after multiplying, per sample, the scores of the
    // items listed in the filter dataset (a sparse dataset over the layer's items) by 0, or by the dataset's float values
    // when bUseValues is set — the device-side form of NNRecsGenerator::generateRecs (utils/NNRecsGenerator.cpp:132-150).
    // Passing the input dataset drops the items a sample already has.
    // The same with the filter as device-resident CSR arrays (row position + b of the arrays filters batch row b; pMul NULL =
    // every listed unit is multiplied by 0): what NNRecsGenerator::generateRecs does with its SamplesFilter, on the device.
    void CalculateFilteredTopK(const string& layer, uint32_t k, const uint64_t* pFilterStart, const uint64_t* pFilterEnd,
                               const uint32_t* pFilterIndex, const NNFloat* pFilterMul, NNFloat* pKey, uint32_t* pValue);
    void CalculateFilteredTopK(const string& layer, uint32_t k, NNDataSetBase* pFilter, GpuBuffer<NNFloat>* pbKey,
                               GpuBuffer<uint32_t>* pbValue, bool bUseValues = false);
    void SetBatch(uint32_t batch);
    // No counterpart in the reference.  With two lanes (the default) consecutive PredictBatch calls alternate between two sets
    // of unit buffers and two device streams: a batch's kernels (and the top-K calls that follow its PredictBatch) overlap
    // with those of the batch before it.  Everything read back through this API waits as needed; a device pointer obtained
    // from GetUnitBuffer belongs to the batch predicted last.  One lane restores single buffers; three or four (at most
    // DSX_MAX_LANES) let consecutive batches take turns on as many sets.
    bool SetLanes(uint32_t lanes);
    // No counterpart in the reference.  By default a wide output layer that feeds nothing else is not computed by PredictBatch
    // but together with the CalculateTopK / CalculateFilteredTopK that follows, without storing its result; GetUnitBuffer and
    // GetUnits compute it on demand.  SetDeferredOutput(false) makes PredictBatch store every layer, as the reference does.
    bool SetDeferredOutput(bool bDefer);
    // No counterpart in the reference.  SetSplitProducts(true): dense layers wide enough for the tiled kernel (at least two
    // 128 x 128 tiles per compute unit) form every fp32 product from six bf16 matrix instructions (dsx_fc_forward_split): sums as
    // close to the exact ones as fp32 multiplication gives, not bit-identical to it, about 1.5 times as fast; the weights of those
    // layers are kept a second time as bf16 planes (1.5 times their size).  A caller
    // that writes weights through NNWeight::GetWeightBuffer calls it again afterwards.  Off by default.
    bool SetSplitProducts(bool bSplit);
    uint32_t GetLanes() const { return _lanes; }
    uint32_t GetLane() const { return _lane; }
    void Randomize();                           // every connection back to its starting values (engine/NNNetwork.cpp:675-679)
    void SetPosition(uint32_t position);
    void SetShuffleIndices(bool bShuffleIndices);
    void SetCPUValidate(bool bValidate);
    bool SaveNetCDF(const string& fname);

    unsigned int GetBatch() const;
    uint32_t GetExamples() const;
    uint32_t GetPosition() const;
    NNWeight* GetWeight(const string& inputLayer, const string& outputLayer) const;
    uint64_t GetBufferSize(const string& layer) const;
    NNLayer* GetLayer(const string& layer) const;
    vector<const NNLayer*>::iterator GetLayers(NNLayer::Kind layerKind, vector<const NNLayer*>& layers) const;
    vector<string> GetLayers() const;
    const string& GetName() const;
    bool GetDebugLevel() const { return _verbose; }
    void SetDebugLevel(bool verbose) { _verbose = verbose; }

    NNFloat* GetUnitBuffer(const string& layer);
    NNFloat* GetWeightBuffer(const string& inputLayer, const string& outputLayer);
};

ostream& operator<<(ostream& out, NNNetwork::Kind& k);

struct NNNetworkDescriptor {
    string _name;
    NNNetwork::Kind _kind;
    ErrorFunction _errorFunction;
    vector<NNLayerDescriptor> _vLayerDescriptor;
    vector<NNWeightDescriptor> _vWeightDescriptor;
    bool _bShuffleIndices;
    NNFloat _decay;
    uint32_t _maxout_k;
    NNFloat _LRN_k;
    uint32_t _LRN_n;
    NNFloat _LRN_alpha;
    NNFloat _LRN_beta;
    NNFloat _RELUSlope;
    NNFloat _ELUAlpha;
    NNFloat _SELULambda;
    bool _bSparsenessPenalty;
    NNFloat _sparsenessPenalty_p;
    NNFloat _sparsenessPenalty_beta;
    bool _bDenoising;
    NNFloat _denoising_p;
    NNFloat _deltaBoost_one;
    NNFloat _deltaBoost_zero;
    NNFloat _SMCE_oneTarget;
    NNFloat _SMCE_zeroTarget;
    NNFloat _SMCE_oneScale;
    NNFloat _SMCE_zeroScale;
    string _checkpoint_name;
    int32_t _checkpoint_interval;
    int32_t _checkpoint_epochs;
    bool _bConvLayersCalculated;
    NNNetworkDescriptor();
};

// Reads a network file with the reference's attribute and variable names (engine/NNNetwork.cpp:3761-4057).
// Returns NULL after printing a message when the file cannot be read.  Caller owns the network.
NNNetwork* LoadNeuralNetworkNetCDF(const string& fname, const uint32_t batch = DefaultBatch);
// Builds a network from an in-memory descriptor (the reference only constructs networks through its file loaders).
NNNetwork* CreateNeuralNetwork(NNNetworkDescriptor& d, const uint32_t batch = DefaultBatch);
bool SaveNeuralNetworkNetCDF(const NNNetwork& net, const string& fname);
// Descriptor-level file I/O, usable without a GPU.
bool LoadNNNetworkDescriptorNetCDF(const string& fname, NNNetworkDescriptor& nd);
bool SaveNNNetworkDescriptorNetCDF(const string& fname, const NNNetworkDescriptor& nd);
// Reads a network definition in JSON (engine/NNNetwork.cpp:2792-3760): "N": "auto" layers take their dimensions from the
// data set of the same name in vDataSet; weights are initialised by each layer's "WeightInit" scheme from the seed given to
// GpuContext::SetRandomSeed.  Returns NULL after printing a message when the file does not parse or names an unknown key.
NNNetwork* LoadNeuralNetworkJSON(const string& fname, const uint32_t batch, const vector<NNDataSetBase*>& vDataSet);
bool LoadNNNetworkDescriptorJSON(const string& fname, NNNetworkDescriptor& nd, const vector<NNDataSetBase*>& vDataSet);

#endif
