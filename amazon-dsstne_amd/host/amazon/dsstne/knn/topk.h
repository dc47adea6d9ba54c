// topk.h — padded top-K of the KNN module (reference: knn/topk.h:73): rows of pitch `width`, the last widthPadding
// columns are not candidates.
#ifndef DSSTNE_AMD_KNN_TOPK_H
#define DSSTNE_AMD_KNN_TOPK_H

#include <cstdint>

typedef float NNFloat;

void kCalculateTopK(NNFloat* pOutput, NNFloat* pKey, uint32_t* pValue, uint32_t batch, uint32_t width, uint32_t widthPadding, uint32_t k);

#endif
