// DsstneContext.h — owns the device context and one network for an embedding process (the JNI / serving entry point of
// the reference, runtime/DsstneContext.h:32-69).  One context per process.
#ifndef DSSTNE_AMD_DSSTNECONTEXT_H
#define DSSTNE_AMD_DSSTNECONTEXT_H

#include "amazon/dsstne/engine/GpuTypes.h"
#include "amazon/dsstne/engine/NNTypes.h"

class DsstneContext {
private:
    static const int ALL = -1;
    const std::string networkFilename;
    const uint32_t batchSize;
    const uint32_t maxK;
    // one set per lane of the network: the results of the batch before the current one stay readable while the current runs
    std::map<string, GpuBuffer<NNFloat>*> dOutputScores[DSX_MAX_LANES];
    std::map<string, GpuBuffer<uint32_t>*> dOutputIndexes[DSX_MAX_LANES];
    std::vector<NNDataSetBase*> ownedDataSets;

public:
    DsstneContext(const std::string& networkFilename, uint32_t batchSize, int maxK = ALL);
    ~DsstneContext();
    NNNetwork* getNetwork() const;
    // Creates empty datasets for the input layers, binds them and runs one prediction so that every buffer exists;
    // afterwards callers only refill the same dataset objects (LoadSparseData / LoadDenseData) and predict.
    void initInputLayerDataSets(const std::vector<NNDataSetDescriptor> datasetDescriptors);
    GpuBuffer<NNFloat>* getOutputScoresBuffer(const std::string& layerName);     // throws std::out_of_range for an unknown layer
    GpuBuffer<uint32_t>* getOutputIndexesBuffer(const std::string& layerName);
    // the same for a given lane: the batch before the current one left its results in the buffers of the lane before the current one
    GpuBuffer<NNFloat>* getOutputScoresBuffer(const std::string& layerName, int lane) { return dOutputScores[lane % DSX_MAX_LANES].at(layerName); }
    GpuBuffer<uint32_t>* getOutputIndexesBuffer(const std::string& layerName, int lane) { return dOutputIndexes[lane % DSX_MAX_LANES].at(layerName); }

    static DsstneContext* fromPtr(long ptr)
    {
        DsstneContext* dc = (DsstneContext*)ptr;
        if (dc == nullptr) throw std::runtime_error("Cannot convert nullptr to DsstneContext");
        return dc;
    }
};

#endif
