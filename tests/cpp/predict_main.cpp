// The reference's C++ specification of the embedding path, java/src/test/native/main.cpp:92-191, re-typed against this
// build's headers: DsstneContext -> input layer descriptors -> initInputLayerDataSets -> LoadSparseData -> SetPosition(0) ->
// PredictBatch -> raw kCalculateTopK on GetUnitBuffer("Output").  Prints one line per sample: "row<TAB>index:score,...".
//   predict_main <network.nc> <inputs.txt> <batch> <k>
// inputs.txt: one line per sample, space-separated item indexes.
#include <fstream>
#include <sstream>

#include "amazon/dsstne/engine/DsstneContext.h"
#include "amazon/dsstne/engine/GpuTypes.h"
#include "amazon/dsstne/engine/NNLayer.h"
#include "amazon/dsstne/engine/NNNetwork.h"
#include "amazon/dsstne/engine/NNTypes.h"

using namespace std;

int main(int argc, char** argv)
{
    if (argc < 5) {
        printf("usage: predict_main network.nc inputs.txt batch k\n");
        return 2;
    }
    const string networkFile = argv[1], inputFile = argv[2];
    const uint32_t batchSize = (uint32_t)atoi(argv[3]), k = (uint32_t)atoi(argv[4]);
    const float sparseDensity = 0.09f;

    DsstneContext dc(networkFile, batchSize);
    NNNetwork* network = dc.getNetwork();
    cout << "predict_main: loaded network " << network->GetName() << endl;

    vector<const NNLayer*> inputLayers;
    vector<NNDataSetDescriptor> datasets;
    for (auto it = network->GetLayers(NNLayer::Kind::Input, inputLayers); it != inputLayers.end(); ++it) {
        const NNLayer* layer = *it;
        NNDataSetDescriptor desc;
        uint32_t x, y, z, w;
        tie(x, y, z, w) = layer->GetDimensions();
        desc._dim = NNDataSetDimensions(x, y, z);
        desc._name = layer->GetDataSetName();
        desc._dataType = NNDataSetEnums::DataType::Int;
        desc._attributes = NNDataSetEnums::Attributes::Sparse;
        desc._examples = network->GetBatch();
        desc._sparseDensity = sparseDensity;
        datasets.push_back(desc);
    }
    dc.initInputLayerDataSets(datasets);

    const NNLayer* inputLayer = network->GetLayer("Input");
    uint32_t x, y, z, w;
    tie(x, y, z, w) = inputLayer->GetDimensions();
    size_t sparseDataLength = (size_t)(((float)(x * y * z * batchSize)) * sparseDensity);
    NNDataSetBase* inputDataset = inputLayer->GetDataSet();

    vector<uint64_t> sparseStart(batchSize, 0), sparseEnd(batchSize, 0);
    vector<uint32_t> sparseIndex(sparseDataLength, 0);
    vector<int> sparseData(sparseDataLength, 0);
    ifstream in(inputFile);
    string line;
    uint32_t row = 0;
    uint64_t pos = 0;
    while (row < batchSize && getline(in, line)) {
        sparseStart[row] = pos;
        stringstream ss(line);
        uint32_t idx;
        while (ss >> idx) {
            sparseIndex[pos] = idx;
            sparseData[pos] = 1;
            ++pos;
        }
        sparseEnd[row] = pos;
        ++row;
    }
    for (; row < batchSize; ++row) sparseStart[row] = sparseEnd[row] = pos;
    inputDataset->LoadSparseData(sparseStart.data(), sparseEnd.data(), sparseData.data(), sparseIndex.data());

    GpuBuffer<NNFloat> outputScores(k * batchSize, false, true);      // managed, like the cudaMallocManaged buffers of main.cpp:147-150
    GpuBuffer<uint32_t> outputIndexes(k * batchSize, false, true);

    network->SetPosition(0);
    network->PredictBatch();
    NNFloat* dUnitBuffer = network->GetUnitBuffer("Output");
    const NNLayer* outputLayer = network->GetLayer("Output");
    tie(x, y, z, w) = outputLayer->GetDimensions();
    kCalculateTopK(dUnitBuffer, outputScores._pDevData, outputIndexes._pDevData, batchSize, x * y * z, k);
    outputScores.Download();   // waits for the kernel; managed memory is then readable from the host

    for (size_t i = 0; i < batchSize; ++i) {
        printf("%zu\t", i);
        for (size_t j = 0; j < k; ++j) printf("%u:%.9g,", outputIndexes._pDevData[i * k + j], outputScores._pDevData[i * k + j]);
        printf("\n");
    }
    return 0;
}
