// NetCDFhelper.h — text samples -> sparse dataset files for the prediction tools (reference: utils/NetCDFhelper.h:36-161).
// Index files are "label<TAB>index" lines; sample files are "sample<TAB>feature[,value]:feature[,value]..." lines.
// The dataset files are written in the classic NetCDF container (see NcClassic.h) with the reference's names.
#ifndef DSSTNE_AMD_NETCDFHELPER_H
#define DSSTNE_AMD_NETCDFHELPER_H

#include <iostream>
#include <map>
#include <string>
#include <unordered_map>
#include <vector>

// Reads "label<TAB>index" lines into labelsToIndices.  false on a malformed line, a repeated label or a read error.
bool loadIndex(std::unordered_map<std::string, unsigned int>& labelsToIndices, std::istream& inputStream, std::ostream& outputStream);
bool loadIndexFromFile(std::unordered_map<std::string, unsigned int>& labelsToIndices, const std::string& inputFile,
                       std::ostream& outputStream);
void exportIndex(std::unordered_map<std::string, unsigned int>& mLabelToIndex, std::string indexFileName);

// One pass over a samples stream.  Unknown samples get the next free index; unknown features are added when
// enableFeatureIndexUpdates is set and skipped otherwise.  mSignals / mSignalValues: sample index -> features / values.
bool parseSamples(std::istream& inputStream, const bool enableFeatureIndexUpdates, std::unordered_map<std::string, unsigned int>& mFeatureIndex,
                  std::unordered_map<std::string, unsigned int>& mSampleIndex, bool& featureIndexUpdated, bool& sampleIndexUpdated,
                  std::map<unsigned int, std::vector<unsigned int>>& mSignals, std::map<unsigned int, std::vector<float>>& mSignalValues,
                  std::ostream& outputStream);

// All files of samplesPath (a file or a directory) -> CSR arrays ordered by sample index.
bool importSamplesFromPath(const std::string& samplesPath, const bool enableFeatureIndexUpdates,
                           std::unordered_map<std::string, unsigned int>& mFeatureIndex,
                           std::unordered_map<std::string, unsigned int>& mSampleIndex, bool& featureIndexUpdated, bool& sampleIndexUpdated,
                           std::vector<unsigned int>& vSparseStart, std::vector<unsigned int>& vSparseEnd,
                           std::vector<unsigned int>& vSparseIndex, std::vector<float>& vSparseData, std::ostream& outputStream);

// importSamplesFromPath + export of whichever index changed.
bool generateNetCDFIndexes(const std::string& samplesPath, const bool enableFeatureIndexUpdates, const std::string& outFeatureIndexFileName,
                           const std::string& outSampleIndexFileName, std::unordered_map<std::string, unsigned int>& mFeatureIndex,
                           std::unordered_map<std::string, unsigned int>& mSampleIndex, std::vector<unsigned int>& vSparseStart,
                           std::vector<unsigned int>& vSparseEnd, std::vector<unsigned int>& vSparseIndex, std::vector<float>& vSparseData,
                           std::ostream& outputStream);

// One sparse dataset per file, width = maxFeatureIndex rounded up to a multiple of 128: analog (float values) ...
void writeNetCDFFile(std::vector<unsigned int>& vSparseStart, std::vector<unsigned int>& vSparseEnd, std::vector<unsigned int>& vSparseIndex,
                     std::vector<float>& vSparseValue, std::string fileName, std::string datasetName, unsigned int maxFeatureIndex);
// ... or Boolean (indices only).
void writeNetCDFFile(std::vector<unsigned int>& vSparseStart, std::vector<unsigned int>& vSparseEnd, std::vector<unsigned int>& vSparseIndex,
                     std::string fileName, std::string datasetName, unsigned int maxFeatureIndex);

unsigned int roundUpMaxIndex(unsigned int maxFeatureIndex);
unsigned int align(size_t size);

#endif
