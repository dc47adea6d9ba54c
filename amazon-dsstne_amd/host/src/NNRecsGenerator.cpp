// NNRecsGenerator.cpp — reference: utils/NNRecsGenerator.cpp:45-244 (single-process path).
#include "amazon/dsstne/utils/NNRecsGenerator.h"

#include <algorithm>

#include "amazon/dsstne/utils/Filters.h"

using namespace std;

const string NNRecsGenerator::DEFAULT_LAYER_RECS_GEN_LABEL = "Output";
const string NNRecsGenerator::DEFAULT_SCORE_PRECISION = "4.3f";
const unsigned int NNRecsGenerator::TOPK_SCALAR = 5;   // the kernel is asked for 5K, the first K are written (utils/NNRecsGenerator.cpp:35,150)

NNRecsGenerator::NNRecsGenerator(unsigned int xBatchSize, unsigned int xK, unsigned int xOutputBufferSize, const string& layer,
                                 const string& precision)
    : pbKey(new GpuBuffer<NNFloat>((size_t)xBatchSize * xK * TOPK_SCALAR, true)),
      pbUIValue(new GpuBuffer<unsigned int>((size_t)xBatchSize * xK * TOPK_SCALAR, true)), recsGenLayerLabel(layer), scorePrecision(precision)
{
    (void)xOutputBufferSize;   // no host copy of the output layer is needed
}

void NNRecsGenerator::generateRecs(NNNetwork* xNetwork, unsigned int xK, const FilterConfig* xFilterSet, const vector<string>& xCustomerIndex,
                                   const vector<string>& xFeatureIndex)
{
    const uint32_t lBatch = std::min<uint32_t>(xNetwork->GetBatch(), xNetwork->GetExamples() - xNetwork->GetPosition());
    const uint32_t lPosition = xNetwork->GetPosition();
    const NNLayer* pLayer = xNetwork->GetLayer(recsGenLayerLabel);
    if (!pLayer) return;
    uint32_t x, y, z, w;
    std::tie(x, y, z, w) = pLayer->GetDimensions();
    const uint32_t width = x * y * z * w;
    const uint32_t kk = std::min<uint32_t>(xK * TOPK_SCALAR, 256u);
    if (kk > width || (size_t)lBatch * kk > pbKey->_length) {
        printf("NNRecsGenerator::generateRecs: k = %u does not fit layer %s or the result buffers.\n", xK, recsGenLayerLabel.c_str());
        return;
    }
    // The reference copies the output rows to the host, multiplies the filtered items there, uploads and runs the top-K
    // (utils/NNRecsGenerator.cpp:138-150); here the filter is applied on the device while the scores are examined.
    SamplesFilter* sf = xFilterSet ? xFilterSet->getSamplesFilter() : NULL;
    if (sf && sf->samples() >= lPosition + lBatch) {
        const uint64_t *fs, *fe;
        const uint32_t* fi;
        const NNFloat* fm;
        sf->deviceArrays(&fs, &fe, &fi, &fm);
        xNetwork->CalculateFilteredTopK(recsGenLayerLabel, kk, fs, fe, fi, fm, pbKey->_pDevData, pbUIValue->_pDevData);
    } else {
        xNetwork->CalculateFilteredTopK(recsGenLayerLabel, kk, NULL, NULL, NULL, NULL, pbKey->_pDevData, pbUIValue->_pDevData);
    }
    pbKey->Download();
    pbUIValue->Download();
    const NNFloat* pKey = pbKey->_pSysData;
    const unsigned int* pIndex = pbUIValue->_pSysData;

    const string fileName = xFilterSet ? xFilterSet->getOutputFileName() : string("recs");
    FILE* fp = fopen(fileName.c_str(), "a");
    if (!fp) {
        printf("NNRecsGenerator::generateRecs: cannot open %s\n", fileName.c_str());
        return;
    }
    const string strFormat = "%s,%" + scorePrecision + ":";
    for (uint32_t j = 0; j < lBatch; j++) {
        fprintf(fp, "%s%c", xCustomerIndex[lPosition + j].c_str(), '\t');
        for (uint32_t r = 0; r < xK && r < kk; ++r) {
            const size_t bufferPos = (size_t)j * kk + r;
            const unsigned int finalIndex = pIndex[bufferPos];
            if (finalIndex < xFeatureIndex.size()) fprintf(fp, strFormat.c_str(), xFeatureIndex[finalIndex].c_str(), pKey[bufferPos]);
        }
        fprintf(fp, "\n");
    }
    fclose(fp);
}
