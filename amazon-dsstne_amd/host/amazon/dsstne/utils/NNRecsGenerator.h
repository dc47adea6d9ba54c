// NNRecsGenerator.h — filtered top-K recommendations of one predicted batch, written as text (reference:
// utils/NNRecsGenerator.h:26-53).  The reference copies the output layer to the host, multiplies on the CPU, uploads and
// sorts; here the filter is applied inside the device top-K kernel and only batch x 5K (score, index) pairs come back.
#ifndef DSSTNE_AMD_NNRECSGENERATOR_H
#define DSSTNE_AMD_NNRECSGENERATOR_H

#include <memory>
#include <string>
#include <vector>

#include "amazon/dsstne/engine/NNTypes.h"

class FilterConfig;
class NNNetwork;

class NNRecsGenerator {
    std::unique_ptr<GpuBuffer<NNFloat>> pbKey;
    std::unique_ptr<GpuBuffer<unsigned int>> pbUIValue;
    std::string recsGenLayerLabel;
    std::string scorePrecision;

public:
    static const std::string DEFAULT_LAYER_RECS_GEN_LABEL;
    static const unsigned int TOPK_SCALAR;
    static const std::string DEFAULT_SCORE_PRECISION;

    NNRecsGenerator(unsigned int xBatchSize, unsigned int xK, unsigned int xOutputBufferSize,
                    const std::string& layer = DEFAULT_LAYER_RECS_GEN_LABEL, const std::string& precision = DEFAULT_SCORE_PRECISION);

    // Appends one line per sample of the current batch to the filter set's output file:
    // "sample<TAB>item,score:item,score:...:" with the first topK of the top 5*topK filtered items.
    void generateRecs(NNNetwork* network, unsigned int topK, const FilterConfig* filters, const std::vector<std::string>& customerIndex,
                      const std::vector<std::string>& featureIndex);
};

#endif
