// predict — recommendations from a trained network for a text file of samples (reference: utils/Predict.cpp:60-276).
//
// Same flags and the same steps as the reference tool: feature index -> samples text to a sparse dataset file -> LoadNetCDF ->
// LoadNeuralNetworkNetCDF -> per batch PredictBatch + NNRecsGenerator::generateRecs (filtered top-K, written as
// "sample<TAB>item,score:item,score:...").  One process, one GPU; the network and dataset files are classic NetCDF (NcClassic.h).
#include <chrono>
#include <iostream>
#include <string>
#include <unordered_map>
#include <vector>

#include "amazon/dsstne/engine/GpuTypes.h"
#include "amazon/dsstne/engine/NNTypes.h"
#include "amazon/dsstne/utils/Filters.h"
#include "amazon/dsstne/utils/NNRecsGenerator.h"
#include "amazon/dsstne/utils/NetCDFhelper.h"
#include "amazon/dsstne/utils/Utils.h"

using namespace std;

static void printUsagePredict()
{
    cout << "Predict: Generates predictions from a trained neural network given a signals/input dataset." << endl;
    cout << "Usage: predict -d <dataset_name> -n <network_file> -r <input_text_file> -i <input_feature_index> -o <output_feature_index> "
            "-f <filters_file> -s <recs_file> [-b <batch_size>] [-k <num_recs>] [-l layer] [-p score_precision]"
         << endl;
    cout << "    -b batch_size: (default = 1024) the number of input rows to process in a batch." << endl;
    cout << "    -d dataset_name: (required) name of the dataset; \"_input\" is appended, as the network's input layer expects." << endl;
    cout << "    -f filters_file: (required) samples filter file or directory: sample<TAB>item[,multiplier]:item..." << endl;
    cout << "    -i input_feature_index: (required) feature<TAB>index file of the network's input features." << endl;
    cout << "    -k num_recs: (default = 100, below 128) predictions per sample, sorted by score." << endl;
    cout << "    -l layer: (default = Output) the network layer to take predictions from." << endl;
    cout << "    -n network_file: (required) the trained network (classic NetCDF)." << endl;
    cout << "    -o output_feature_index: (required) feature<TAB>index file that names the units of the prediction layer." << endl;
    cout << "    -p score_precision: (default = 4.3f) printf precision of the scores." << endl;
    cout << "    -r input_text_file: (required) the samples: sample<TAB>feature[,value]:feature[,value]..." << endl;
    cout << "    -s recs_file: (required) where the recommendations are written." << endl;
}

static string requiredFile(int argc, char** argv, const string& flag, const string& what)
{
    string name = getRequiredArgValue(argc, argv, flag, what + " is not specified.", &printUsagePredict);
    if (!fileExists(name)) {
        cout << "Error: Cannot read " << what << ": " << name << endl;
        exit(1);
    }
    return name;
}

int main(int argc, char** argv)
{
    if (isArgSet(argc, argv, "-h")) {
        printUsagePredict();
        return 1;
    }
    const string dataSetName = getRequiredArgValue(argc, argv, "-d", "dataset_name is not specified.", &printUsagePredict) + INPUT_DATASET_SUFFIX;
    const string filtersFileName = requiredFile(argc, argv, "-f", "filter file");
    const string inputIndexFileName = requiredFile(argc, argv, "-i", "input features index file");
    const string networkFileName = requiredFile(argc, argv, "-n", "network file");
    const string outputIndexFileName = requiredFile(argc, argv, "-o", "output features index file");
    const string samplesFileName = requiredFile(argc, argv, "-r", "input_text_file");
    const string recsOutputFileName = getRequiredArgValue(argc, argv, "-s", "filename to put the output recs to.", &printUsagePredict);
    const unsigned int batchSize = (unsigned int)stoi(getOptionalArgValue(argc, argv, "-b", "1024"));
    const unsigned int topK = (unsigned int)stoi(getOptionalArgValue(argc, argv, "-k", "100"));
    if (topK >= 128) {
        cout << "Error :Optimized topk Only works for top 128 . " << topK << " is greater" << endl;
        return 1;
    }
    const string scoreFormat = getOptionalArgValue(argc, argv, "-p", NNRecsGenerator::DEFAULT_SCORE_PRECISION);
    const string recsGenLayerLabel = getOptionalArgValue(argc, argv, "-l", NNRecsGenerator::DEFAULT_LAYER_RECS_GEN_LABEL);

    getGpu().Startup(argc, argv);
    getGpu().SetRandomSeed(FIXED_SEED);
    const auto preProcessingStart = chrono::steady_clock::now();

    unordered_map<string, unsigned int> mInput;
    cout << "Loading input feature index from: " << inputIndexFileName << endl;
    if (!loadIndexFromFile(mInput, inputIndexFileName, cout)) return 1;

    // samples text -> sparse dataset file next to the working directory, named so that training files are not overwritten
    unordered_map<string, unsigned int> mSignals;
    const string dataSetFilesPrefix = dataSetName + "_predict";
    const string inputNetCDFFileName = dataSetFilesPrefix + NETCDF_FILE_EXTENTION;
    {
        vector<unsigned int> vSparseStart, vSparseEnd, vSparseIndex;
        vector<float> vSparseData;
        if (!generateNetCDFIndexes(samplesFileName, false, dataSetFilesPrefix + ".featuresIndex", dataSetFilesPrefix + ".samplesIndex", mInput, mSignals,
                                   vSparseStart, vSparseEnd, vSparseIndex, vSparseData, cout))
            return 1;
        writeNetCDFFile(vSparseStart, vSparseEnd, vSparseIndex, inputNetCDFFileName, dataSetName, (unsigned int)mInput.size());
    }
    cout << "Number of network input nodes: " << mInput.size() << endl;
    cout << "Number of entries to generate predictions for: " << mSignals.size() << endl;

    vector<NNDataSetBase*> vDataSetInput = LoadNetCDF(inputNetCDFFileName);
    NNNetwork* pNetwork = LoadNeuralNetworkNetCDF(networkFileName, batchSize);
    pNetwork->LoadDataSets(vDataSetInput);

    vector<string> vSignals(mSignals.size());
    for (const auto& kv : mSignals) vSignals[kv.second] = kv.first;

    unordered_map<string, unsigned int> mOutput;
    cout << "Loading output feature index from: " << outputIndexFileName << endl;
    if (!loadIndexFromFile(mOutput, outputIndexFileName, cout)) return 1;
    unsigned int maxOutputIndex = 0;
    for (const auto& kv : mOutput) maxOutputIndex = max(maxOutputIndex, kv.second);
    vector<string> vOutput(mOutput.empty() ? 0 : maxOutputIndex + 1);
    for (const auto& kv : mOutput) vOutput[kv.second] = kv.first;
    FilterConfig* vFilterSet = loadFilters(filtersFileName, recsOutputFileName, mOutput, mSignals);
    mInput.clear();
    mOutput.clear();
    mSignals.clear();
    cout << "Total time for loading network and data is: " << elapsed_seconds(preProcessingStart, chrono::steady_clock::now()) << endl;

    if (!pNetwork->GetLayer(recsGenLayerLabel)) {
        cout << "Error: the network has no layer " << recsGenLayerLabel << endl;
        return 1;
    }
    NNRecsGenerator* nnRecsGenerator =
        new NNRecsGenerator(pNetwork->GetBatch(), topK, (unsigned int)pNetwork->GetBufferSize(recsGenLayerLabel), recsGenLayerLabel, scoreFormat);
    const auto recsGenerationStart = chrono::steady_clock::now();
    for (unsigned long long pos = 0; pos < pNetwork->GetExamples(); pos += pNetwork->GetBatch()) {
        cout << "Predicting from position " << pos << endl;
        pNetwork->SetPosition((uint32_t)pos);
        pNetwork->PredictBatch();
        nnRecsGenerator->generateRecs(pNetwork, topK, vFilterSet, vSignals, vOutput);
    }
    cout << "Total time for Generating recs for " << pNetwork->GetExamples() << " was "
         << elapsed_seconds(recsGenerationStart, chrono::steady_clock::now()) << endl;

    delete nnRecsGenerator;
    delete vFilterSet;
    delete pNetwork;
    for (auto p : vDataSetInput) delete p;
    getGpu().Shutdown();
    return 0;
}
