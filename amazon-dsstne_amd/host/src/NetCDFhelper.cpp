// NetCDFhelper.cpp — reference: utils/NetCDFhelper.cpp:36-420 (index files, sample text parsing, single-dataset files).
#include "amazon/dsstne/utils/NetCDFhelper.h"

#include <cerrno>
#include <cstring>
#include <fstream>
#include <stdexcept>

#include "NcClassic.h"
#include "amazon/dsstne/engine/NNEnum.h"
#include "amazon/dsstne/utils/Utils.h"

using namespace std;

bool loadIndex(unordered_map<string, unsigned int>& labelsToIndices, istream& inputStream, ostream& outputStream)
{
    // "label<TAB>index" per line; exactly one tab, a non-empty label, and every line must bring a label not seen before
    // (utils/NetCDFhelper.cpp:36-65: the reference compares lines read with entries added).
    const size_t before = labelsToIndices.size();
    size_t lines = 0;
    for (string line; getline(inputStream, line);) {
        ++lines;
        const size_t tab = line.find('\t');
        const bool oneTab = tab != string::npos && line.find('\t', tab + 1) == string::npos;
        if (!oneTab || tab == 0) {
            outputStream << "Error: line " << lines << " contains invalid data" << endl;
            return false;
        }
        labelsToIndices[line.substr(0, tab)] = (unsigned int)strtol(line.c_str() + tab + 1, nullptr, 10);
    }
    const size_t added = labelsToIndices.size() - before;
    outputStream << "Number of lines processed: " << lines << endl << "Number of entries added to index: " << added << endl;
    if (added != lines) {
        outputStream << "Error: Number of entries added to index not equal to number of lines processed" << endl;
        return false;
    }
    if (inputStream.bad()) {
        outputStream << "Error: " << strerror(errno) << endl;
        return false;
    }
    return true;
}

bool loadIndexFromFile(unordered_map<string, unsigned int>& labelsToIndices, const string& inputFile, ostream& outputStream)
{
    ifstream inputStream(inputFile);
    if (!inputStream.is_open()) {
        outputStream << "Error: Failed to open index file" << endl;
        return false;
    }
    return loadIndex(labelsToIndices, inputStream, outputStream);
}

void exportIndex(unordered_map<string, unsigned int>& mLabelToIndex, string indexFileName)
{
    ofstream out(indexFileName);
    for (const auto& kv : mLabelToIndex) out << kv.first << "\t" << kv.second << endl;
}

bool parseSamples(istream& inputStream, const bool enableFeatureIndexUpdates, unordered_map<string, unsigned int>& mFeatureIndex,
                  unordered_map<string, unsigned int>& mSampleIndex, bool& featureIndexUpdated, bool& sampleIndexUpdated,
                  map<unsigned int, vector<unsigned int>>& mSignals, map<unsigned int, vector<float>>& mSignalValues, ostream& outputStream)
{
    string line;
    int lineNumber = 0;
    while (getline(inputStream, line)) {
        lineNumber++;
        if (line.empty()) continue;
        const size_t tab = line.find('\t');
        if (tab == string::npos) {
            outputStream << "Warning: Skipping over malformed line (" << line << ") at line " << lineNumber << endl;
            continue;
        }
        const string sampleLabel = line.substr(0, tab);
        const string dataString = line.substr(tab + 1);

        unsigned int sampleIndex;
        auto sit = mSampleIndex.find(sampleLabel);
        if (sit != mSampleIndex.end()) {
            sampleIndex = sit->second;
        } else {
            sampleIndex = (unsigned int)mSampleIndex.size();
            mSampleIndex[sampleLabel] = sampleIndex;
            sampleIndexUpdated = true;
        }

        vector<unsigned int> signals;
        vector<float> signalValue;
        for (const string& dataPoint : split(dataString, ':')) {
            vector<string> dataElems = split(dataPoint, ',');
            if (dataElems.empty() || dataElems[0].empty()) continue;
            if (dataElems.size() > 2) {
                outputStream << "Warning: Data point [" << dataPoint << "] at line " << lineNumber << " has more than 1 value for feature (actual value: "
                             << dataElems.size() << "). Keeping the first value and ignoring subsequent values." << endl;
            }
            float featureValue = 0.0f;
            if (dataElems.size() > 1) featureValue = stof(dataElems[1]);   // throws on garbage, like the reference
            unsigned int featureIndex;
            auto fit = mFeatureIndex.find(dataElems[0]);
            if (fit != mFeatureIndex.end()) {
                featureIndex = fit->second;
            } else if (enableFeatureIndexUpdates) {
                featureIndex = (unsigned int)mFeatureIndex.size();
                mFeatureIndex[dataElems[0]] = featureIndex;
                featureIndexUpdated = true;
            } else {
                continue;   // unknown feature and a frozen index: the data point is dropped
            }
            signals.push_back(featureIndex);
            signalValue.push_back(featureValue);
        }
        // a sample that appears twice keeps its last line (utils/NetCDFhelper.cpp:188-189)
        mSignals[sampleIndex] = signals;
        mSignalValues[sampleIndex] = signalValue;
    }
    if (inputStream.bad()) {
        outputStream << "Error: " << strerror(errno) << endl;
        return false;
    }
    return true;
}

bool importSamplesFromPath(const string& samplesPath, const bool enableFeatureIndexUpdates, unordered_map<string, unsigned int>& mFeatureIndex,
                           unordered_map<string, unsigned int>& mSampleIndex, bool& featureIndexUpdated, bool& sampleIndexUpdated,
                           vector<unsigned int>& vSparseStart, vector<unsigned int>& vSparseEnd, vector<unsigned int>& vSparseIndex,
                           vector<float>& vSparseData, ostream& outputStream)
{
    featureIndexUpdated = false;
    sampleIndexUpdated = false;
    if (!fileExists(samplesPath)) {
        outputStream << "Error: " << samplesPath << " not found." << endl;
        return false;
    }
    // the whole input is buffered so that rows come out in sample-index order whatever the order of the lines
    map<unsigned int, vector<unsigned int>> mSignals;
    map<unsigned int, vector<float>> mSignalValues;
    vector<string> files;
    if (listFiles(samplesPath, false, files) == 0) {
        outputStream << "Indexing " << files.size() << " files" << endl;
        for (const string& file : files) {
            outputStream << "\tIndexing file: " << file << endl;
            ifstream inputStream(file);
            if (!inputStream.is_open()) {
                outputStream << "Error: Failed to open index file" << endl;
                return false;
            }
            if (!parseSamples(inputStream, enableFeatureIndexUpdates, mFeatureIndex, mSampleIndex, featureIndexUpdated, sampleIndexUpdated, mSignals,
                              mSignalValues, outputStream))
                return false;
        }
    }
    for (const auto& kv : mSignals) {
        vSparseStart.push_back((unsigned int)vSparseIndex.size());
        const vector<float>& values = mSignalValues[kv.first];
        for (size_t i = 0; i < kv.second.size(); i++) {
            vSparseIndex.push_back(kv.second[i]);
            vSparseData.push_back(values[i]);
        }
        vSparseEnd.push_back((unsigned int)vSparseIndex.size());
    }
    return true;
}

bool generateNetCDFIndexes(const string& samplesPath, const bool enableFeatureIndexUpdates, const string& outFeatureIndexFileName,
                           const string& outSampleIndexFileName, unordered_map<string, unsigned int>& mFeatureIndex,
                           unordered_map<string, unsigned int>& mSampleIndex, vector<unsigned int>& vSparseStart,
                           vector<unsigned int>& vSparseEnd, vector<unsigned int>& vSparseIndex, vector<float>& vSparseData,
                           ostream& outputStream)
{
    bool featureIndexUpdated = false, sampleIndexUpdated = false;
    if (!importSamplesFromPath(samplesPath, enableFeatureIndexUpdates, mFeatureIndex, mSampleIndex, featureIndexUpdated, sampleIndexUpdated,
                               vSparseStart, vSparseEnd, vSparseIndex, vSparseData, outputStream))
        return false;
    if (featureIndexUpdated) {
        exportIndex(mFeatureIndex, outFeatureIndexFileName);
        outputStream << "Exported " << outFeatureIndexFileName << " with " << mFeatureIndex.size() << " entries." << endl;
    }
    if (sampleIndexUpdated) {
        exportIndex(mSampleIndex, outSampleIndexFileName);
        outputStream << "Exported " << outSampleIndexFileName << " with " << mSampleIndex.size() << " entries." << endl;
    }
    return true;
}

unsigned int roundUpMaxIndex(unsigned int maxFeatureIndex) { return ((maxFeatureIndex + 127) >> 7) << 7; }
unsigned int align(size_t size) { return (unsigned int)((size + 127) >> 7) << 7; }

// Attributes and variables of dataset 0 exactly as the reference tool writes them (utils/NetCDFhelper.cpp:332-412); offsets stay
// 32-bit in the file (the dataset reader widens them).
static void writeSparse(const vector<unsigned int>& vSparseStart, const vector<unsigned int>& vSparseEnd, const vector<unsigned int>& vSparseIndex,
                        const vector<float>* pSparseValue, const string& fileName, const string& datasetName, unsigned int maxFeatureIndex)
{
    cout << "Raw max index is: " << maxFeatureIndex << endl;
    maxFeatureIndex = roundUpMaxIndex(maxFeatureIndex);
    cout << "Rounded up max index to: " << maxFeatureIndex << endl;
    try {
        ncc::Writer nc;
        nc.putAttUInt("datasets", 1);
        nc.putAttString("name0", datasetName);
        nc.putAttUInt("attributes0", pSparseValue ? (uint32_t)NNDataSetEnums::Sparse : (uint32_t)(NNDataSetEnums::Sparse + NNDataSetEnums::Boolean));
        nc.putAttUInt("kind0", (uint32_t)NNDataSetEnums::Numeric);
        nc.putAttUInt("dataType0", pSparseValue ? (uint32_t)NNDataSetEnums::Float : (uint32_t)NNDataSetEnums::UInt);
        nc.putAttUInt("dimensions0", 1);
        nc.putAttUInt("width0", maxFeatureIndex);
        const uint32_t examplesDim = nc.addDim("examplesDim0", vSparseStart.size());
        const uint32_t sparseDataDim = nc.addDim("sparseDataDim0", vSparseIndex.size());
        nc.addVar("sparseStart0", ncc::NC_UINT, examplesDim, vSparseStart.data());
        nc.addVar("sparseEnd0", ncc::NC_UINT, examplesDim, vSparseEnd.data());
        nc.addVar("sparseIndex0", ncc::NC_UINT, sparseDataDim, vSparseIndex.data());
        if (pSparseValue) nc.addVar("sparseData0", ncc::NC_FLOAT, sparseDataDim, pSparseValue->data());
        nc.write(fileName);
        cout << "Created NetCDF file " << fileName << " for dataset " << datasetName << endl;
    } catch (exception& e) {
        cout << "Caught exception: " << e.what() << "\n";
        throw runtime_error("Error writing to NetCDF file.");
    }
}

void writeNetCDFFile(vector<unsigned int>& vSparseStart, vector<unsigned int>& vSparseEnd, vector<unsigned int>& vSparseIndex,
                     vector<float>& vSparseValue, string fileName, string datasetName, unsigned int maxFeatureIndex)
{
    writeSparse(vSparseStart, vSparseEnd, vSparseIndex, &vSparseValue, fileName, datasetName, maxFeatureIndex);
}

void writeNetCDFFile(vector<unsigned int>& vSparseStart, vector<unsigned int>& vSparseEnd, vector<unsigned int>& vSparseIndex, string fileName,
                     string datasetName, unsigned int maxFeatureIndex)
{
    writeSparse(vSparseStart, vSparseEnd, vSparseIndex, nullptr, fileName, datasetName, maxFeatureIndex);
}
