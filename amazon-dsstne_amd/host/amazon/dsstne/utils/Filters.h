// Filters.h — per-sample recommendation filters (reference: utils/Filters.h:23-140).
// A sample's filter maps item index -> multiplier (0 when the file lists the item without a value).  Besides the host
// multiply of the reference (applyFilter), the whole filter set can be handed to the GPU once as a CSR matrix so that
// filtering happens inside the top-K kernel and the scores never travel to the host.
#ifndef DSSTNE_AMD_FILTERS_H
#define DSSTNE_AMD_FILTERS_H

#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "amazon/dsstne/engine/GpuTypes.h"

class AbstractFilter {
public:
    virtual ~AbstractFilter() = default;
    virtual void loadFilter(std::unordered_map<std::string, unsigned int>& xMInput, std::unordered_map<std::string, unsigned int>& xMSamples,
                            const std::string& filePath) = 0;
    virtual void applyFilter(float* xArray, int xSamplesIndex) const = 0;
    virtual void applyFilter(float* xArray, int xSamplesIndex, int offset, int width) const = 0;
    virtual std::string getFilterType() const = 0;

protected:
    void updateRecords(float* xArray, const std::unordered_map<int, float>* xFilter) const;
    void updateRecords(float* xArray, const std::unordered_map<int, float>* xFilter, int offset, int width) const;
};

class SamplesFilter : public AbstractFilter {
    std::unique_ptr<std::vector<std::unique_ptr<std::unordered_map<int, float>>>> samplefilters;
    // device copy: CSR over all samples
    std::unique_ptr<GpuBuffer<uint64_t>> pbStart, pbEnd;
    std::unique_ptr<GpuBuffer<uint32_t>> pbIndex;
    std::unique_ptr<GpuBuffer<NNFloat>> pbMul;

    void loadSingleFilter(std::unordered_map<std::string, unsigned int>& xMInput, std::unordered_map<std::string, unsigned int>& xMSamples,
                          std::vector<std::unique_ptr<std::unordered_map<int, float>>>& sampleFilters, const std::string& filePath);

public:
    void loadFilter(std::unordered_map<std::string, unsigned int>& xMInput, std::unordered_map<std::string, unsigned int>& xMSamples,
                    const std::string& filePath) override;
    // Programmatic form of loadFilter: sample -> {item -> multiplier}.
    void setFilters(size_t samples, const std::vector<std::unordered_map<int, float>>& filters);
    void applyFilter(float* xArray, int xSamplesIndex) const override;
    void applyFilter(float* xArray, int xSamplesIndex, int offset, int width) const override;
    std::string getFilterType() const override { return "samplesFilterType"; }

    size_t samples() const { return samplefilters ? samplefilters->size() : 0; }
    // Builds (once) and returns the device CSR arrays; row s is the filter of sample s.
    void deviceArrays(const uint64_t** start, const uint64_t** end, const uint32_t** index, const NNFloat** mul);
};

class FilterConfig {
    std::unique_ptr<SamplesFilter> sampleFilter;
    std::string outputFileName;

public:
    void setOutputFileName(const std::string& xOutputFileName) { outputFileName = xOutputFileName; }
    std::string getOutputFileName() const { return outputFileName; }
    void setSamplesFilter(SamplesFilter* xSampleFilter) { sampleFilter.reset(xSampleFilter); }
    SamplesFilter* getSamplesFilter() const { return sampleFilter.get(); }
    void applySamplesFilter(float* xInput, int xSampleIndex, int offset, int width) const
    {
        if (sampleFilter) sampleFilter->applyFilter(xInput, xSampleIndex, offset, width);
    }
};

// Loads "sample<TAB>item[,value]:item[,value]..." files; the output file is truncated.  Caller owns the result.
FilterConfig* loadFilters(const std::string& samplesFilterFileName, const std::string& outputFileName,
                          std::unordered_map<std::string, unsigned int>& xMInput, std::unordered_map<std::string, unsigned int>& xMSamples);

#endif
