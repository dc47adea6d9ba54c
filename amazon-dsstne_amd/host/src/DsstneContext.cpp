// DsstneContext.cpp — reference: runtime/DsstneContext.cpp:29-124.
#include <stdexcept>

#include "amazon/dsstne/runtime/DsstneContext.h"

namespace {
const int ARGC = 1;
char ARGV0[] = "dsstne-faux-process";
char* ARGV = ARGV0;
const unsigned long SEED = 12134ULL;
}  // namespace

using namespace std;

DsstneContext::DsstneContext(const string& networkFilename, uint32_t batchSize, int maxK)
    : networkFilename(networkFilename), batchSize(batchSize), maxK(maxK)
{
    getGpu().Startup(ARGC, &ARGV);
    getGpu().SetRandomSeed(SEED);
    NNNetwork* network = LoadNeuralNetworkNetCDF(networkFilename, batchSize);
    getGpu().SetNeuralNetwork(network);

    vector<const NNLayer*> outputLayers;
    auto it = network->GetLayers(NNLayer::Kind::Output, outputLayers);
    for (; it != outputLayers.end(); ++it) {
        const string& layerName = (*it)->GetName();
        if (maxK != ALL) {
            if ((*it)->GetNumDimensions() > 1) throw std::runtime_error("topK only supported on 1-D output layers");
            size_t outputBufferLength = (size_t)maxK * batchSize;
            printf("DsstneContext::DsstneContext: Allocating output score and index buffers, each of size %zu for output layer %s\n",
                   outputBufferLength, layerName.c_str());
            for (int lane = 0; lane < DSX_MAX_LANES; lane++) {
                dOutputScores[lane][layerName] = new GpuBuffer<NNFloat>(outputBufferLength, false, false);
                dOutputIndexes[lane][layerName] = new GpuBuffer<uint32_t>(outputBufferLength, false, false);
            }
        }
    }
}

// The buffers of the batch predicted last (the network's current lane).
GpuBuffer<NNFloat>* DsstneContext::getOutputScoresBuffer(const std::string& layerName)
{
    return dOutputScores[getNetwork() ? getNetwork()->GetLane() : 0].at(layerName);
}

GpuBuffer<uint32_t>* DsstneContext::getOutputIndexesBuffer(const std::string& layerName)
{
    return dOutputIndexes[getNetwork() ? getNetwork()->GetLane() : 0].at(layerName);
}

DsstneContext::~DsstneContext()
{
    const string networkName = getNetwork() ? getNetwork()->GetName() : string("<none>");
    for (int lane = 0; lane < DSX_MAX_LANES; lane++) {
        for (const auto& kv : dOutputScores[lane]) delete kv.second;
        for (const auto& kv : dOutputIndexes[lane]) delete kv.second;
        dOutputScores[lane].clear();
        dOutputIndexes[lane].clear();
    }
    delete getNetwork();
    for (auto d : ownedDataSets) delete d;
    ownedDataSets.clear();
    getGpu().Shutdown();
    printf("DsstneContext::~DsstneContext: Destroyed context for network %s\n", networkName.c_str());
}

NNNetwork* DsstneContext::getNetwork() const { return getGpu()._pNetwork; }

void DsstneContext::initInputLayerDataSets(const vector<NNDataSetDescriptor> datasetDescriptors)
{
    vector<NNDataSetBase*> datasets;
    for (const auto& descriptor : datasetDescriptors) {
        NNDataSetBase* dataset = createNNDataSet(descriptor);
        datasets.push_back(dataset);
        ownedDataSets.push_back(dataset);
    }
    NNNetwork* network = getNetwork();
    network->LoadDataSets(datasets);
    network->PredictBatch();
    network->SetPosition(0);
}
