// kernels.h — host-callable launchers with the reference's names and argument orders (engine/kernels.h:16-243), for callers
// that drive kernels on raw device pointers.  Each forwards to the C ABI of libdsx_hip.so.
#ifndef DSSTNE_AMD_KERNELS_H
#define DSSTNE_AMD_KERNELS_H

#include "GpuTypes.h"

void kClearUnit(NNFloat* pUnit, NNFloat* pBias, uint32_t stride, uint32_t batch);
void kClearDualSourceUnit(NNFloat* pUnit, NNFloat* pBias1, NNFloat* pBias2, uint32_t stride, uint32_t batch);
void kClearTripleSourceUnit(NNFloat* pUnit, NNFloat* pBias1, NNFloat* pBias2, NNFloat* pBias3, uint32_t stride, uint32_t batch);
void kClearQuadSourceUnit(NNFloat* pUnit, NNFloat* pBias1, NNFloat* pBias2, NNFloat* pBias3, NNFloat* pBias4, uint32_t stride, uint32_t batch);

void kCalculateSparseZ(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pWeight, uint64_t* pSparseStart, uint64_t* pSparseEnd,
                       uint32_t* pSparseIndex, NNFloat* pDataWeight, NNFloat* pUnit, NNFloat beta);
void kCalculateIndexedSparseZ(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pWeight, uint32_t* pIndex, uint64_t* pSparseStart,
                              uint64_t* pSparseEnd, uint32_t* pSparseIndex, NNFloat* pDataWeight, NNFloat* pUnit, NNFloat beta);
template <typename T>
void kCalculateSparseAnalogZ(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pWeight, uint64_t* pSparseStart, uint64_t* pSparseEnd,
                             uint32_t* pSparseIndex, NNFloat* pDataWeight, T* pSparseData, NNFloat* pUnit, NNFloat beta);
template <typename T>
void kCalculateIndexedSparseAnalogZ(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pWeight, uint32_t* pIndex,
                                    uint64_t* pSparseStart, uint64_t* pSparseEnd, uint32_t* pSparseIndex, NNFloat* pDataWeight, T* pSparseData,
                                    NNFloat* pUnit, NNFloat beta);

void kCalculateSigmoidActivation(NNFloat* pData, uint64_t size);
void kCalculateTanhActivation(NNFloat* pData, uint64_t size);
void kCalculateRELUActivation(NNFloat* pData, uint64_t size);
void kCalculateLRELUActivation(NNFloat* pData, uint64_t size, NNFloat slope);
void kCalculateELUActivation(NNFloat* pData, uint64_t size, NNFloat alpha);
void kCalculateSELUActivation(NNFloat* pData, uint64_t size, NNFloat alpha, NNFloat lambda);
void kCalculateSoftMaxActivation(NNFloat* pData, uint32_t batch, uint32_t stride);

void kAddBuffers(NNFloat* pDest, NNFloat* pSrc, uint64_t size);

void kCalculateTopK(NNFloat* pOutputKey, NNFloat* pKey, uint32_t* pValue, uint32_t batch, uint32_t width, uint32_t k);
void kCalculateTopK(NNFloat* pOutputKey, NNFloat* pOutputValue, NNFloat* pKey, NNFloat* pValue, uint32_t batch, uint32_t width, uint32_t k);
void kCalculateTopK(NNFloat* pOutputKey, uint32_t* pOutputValue, NNFloat* pKey, uint32_t* pValue, uint32_t batch, uint32_t width, uint32_t k);

#endif
