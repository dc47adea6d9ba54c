// Filters.cpp — reference: utils/Filters.cpp:30-216.
#include "amazon/dsstne/utils/Filters.h"

#include <fstream>
#include <iostream>
#include <stdexcept>

#include "amazon/dsstne/utils/Utils.h"

using namespace std;

void AbstractFilter::updateRecords(float* xArray, const unordered_map<int, float>* xFilter) const
{
    if (!xFilter) return;
    for (const auto& kv : *xFilter) xArray[kv.first] = kv.second * xArray[kv.first];
}

void AbstractFilter::updateRecords(float* xArray, const unordered_map<int, float>* xFilter, int offset, int width) const
{
    if (!xFilter) return;
    for (const auto& kv : *xFilter)
        if (kv.first >= offset && kv.first < offset + width) xArray[kv.first - offset] = kv.second * xArray[kv.first - offset];
}

void SamplesFilter::loadSingleFilter(unordered_map<string, unsigned int>& xMInput, unordered_map<string, unsigned int>& xMSamples,
                                     vector<unique_ptr<unordered_map<int, float>>>& sampleFilters, const string& filePath)
{
    ifstream samplesFile(filePath);
    if (!samplesFile.good()) {
        cout << "Unable to read the file " << filePath << endl;
        throw std::invalid_argument("invalid sample filters " + filePath + ", exiting...");
    }
    string line;
    while (getline(samplesFile, line)) {
        // sample<TAB>item[,value]:item[,value]...
        const size_t tab = line.find('\t');
        const string sampleName = line.substr(0, tab);
        auto s = xMSamples.find(sampleName);
        if (s == xMSamples.end()) continue;   // unknown sample: line ignored
        unique_ptr<unordered_map<int, float>> filter(new unordered_map<int, float>());
        if (tab != string::npos) {
            for (const string& entry : split(line.substr(tab + 1), ':')) {
                vector<string> vals = split(entry, ',');
                if (vals.empty()) continue;
                auto item = xMInput.find(vals[0]);
                if (item == xMInput.end()) continue;   // unknown item: entry ignored
                (*filter)[(int)item->second] = vals.size() > 1 ? (float)atof(vals[1].c_str()) : 0.0f;
            }
        }
        sampleFilters[s->second] = std::move(filter);
    }
}

void SamplesFilter::loadFilter(unordered_map<string, unsigned int>& xMInput, unordered_map<string, unsigned int>& xMSamples,
                               const string& filterFilePath)
{
    samplefilters.reset(new vector<unique_ptr<unordered_map<int, float>>>(xMSamples.size()));
    pbStart.reset();
    vector<string> files;
    if (listFiles(filterFilePath, false, files) == 0) {
        cout << "Loading " << files.size() << " filter files" << endl;
        for (auto const& file : files) {
            cout << "\tLoading filter: " << file << endl;
            loadSingleFilter(xMInput, xMSamples, *samplefilters, file);
        }
    }
    cout << "Info:SamplesFilter " << samplefilters->size() << endl;
}

void SamplesFilter::setFilters(size_t samples, const vector<unordered_map<int, float>>& filters)
{
    samplefilters.reset(new vector<unique_ptr<unordered_map<int, float>>>(samples));
    pbStart.reset();
    for (size_t i = 0; i < filters.size() && i < samples; i++)
        (*samplefilters)[i].reset(new unordered_map<int, float>(filters[i]));
}

void SamplesFilter::applyFilter(float* xArray, int xSamplesIndex, int offset, int width) const
{
    updateRecords(xArray, (*samplefilters)[xSamplesIndex].get(), offset, width);
}

void SamplesFilter::applyFilter(float* xArray, int xSamplesIndex) const { updateRecords(xArray, (*samplefilters)[xSamplesIndex].get()); }

void SamplesFilter::deviceArrays(const uint64_t** start, const uint64_t** end, const uint32_t** index, const NNFloat** mul)
{
    if (!pbStart) {
        const size_t n = samples();
        vector<uint64_t> vs(n), ve(n);
        vector<uint32_t> vi;
        vector<NNFloat> vm;
        for (size_t s = 0; s < n; s++) {
            vs[s] = vi.size();
            if ((*samplefilters)[s])
                for (const auto& kv : *(*samplefilters)[s])
                    if (kv.first >= 0) {
                        vi.push_back((uint32_t)kv.first);
                        vm.push_back(kv.second);
                    }
            ve[s] = vi.size();
        }
        pbStart.reset(new GpuBuffer<uint64_t>(n));
        pbEnd.reset(new GpuBuffer<uint64_t>(n));
        pbIndex.reset(new GpuBuffer<uint32_t>(vi.size()));
        pbMul.reset(new GpuBuffer<NNFloat>(vm.size()));
        pbStart->Upload(vs.data());
        pbEnd->Upload(ve.data());
        if (!vi.empty()) {
            pbIndex->Upload(vi.data());
            pbMul->Upload(vm.data());
        }
    }
    *start = pbStart->_pDevData;
    *end = pbEnd->_pDevData;
    *index = pbIndex->_pDevData;
    *mul = pbMul->_pDevData;
}

FilterConfig* loadFilters(const string& samplesFilterFileName, const string& outputFileName, unordered_map<string, unsigned int>& xMInput,
                          unordered_map<string, unsigned int>& xMSamples)
{
    FilterConfig* filterConfig = new FilterConfig();
    SamplesFilter* samplesFilter = new SamplesFilter();
    samplesFilter->loadFilter(xMInput, xMSamples, samplesFilterFileName);
    filterConfig->setSamplesFilter(samplesFilter);
    filterConfig->setOutputFileName(outputFileName);
    FILE* fp = fopen(outputFileName.c_str(), "w");   // start from an empty output file
    if (fp) fclose(fp);
    return filterConfig;
}
