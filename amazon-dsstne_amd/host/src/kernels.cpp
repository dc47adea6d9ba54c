// kernels.cpp — reference-named launchers over the C ABI (see engine/kernels.h of this build).
#include "amazon/dsstne/engine/NNTypes.h"

void kClearUnit(NNFloat* pUnit, NNFloat* pBias, uint32_t stride, uint32_t batch)
{
    dsxFatal(dsx_clear_unit(pUnit, pBias, NULL, NULL, NULL, 1, stride, batch), "kClearUnit");
}
void kClearDualSourceUnit(NNFloat* pUnit, NNFloat* pBias1, NNFloat* pBias2, uint32_t stride, uint32_t batch)
{
    dsxFatal(dsx_clear_unit(pUnit, pBias1, pBias2, NULL, NULL, 2, stride, batch), "kClearDualSourceUnit");
}
void kClearTripleSourceUnit(NNFloat* pUnit, NNFloat* pBias1, NNFloat* pBias2, NNFloat* pBias3, uint32_t stride, uint32_t batch)
{
    dsxFatal(dsx_clear_unit(pUnit, pBias1, pBias2, pBias3, NULL, 3, stride, batch), "kClearTripleSourceUnit");
}
void kClearQuadSourceUnit(NNFloat* pUnit, NNFloat* pBias1, NNFloat* pBias2, NNFloat* pBias3, NNFloat* pBias4, uint32_t stride, uint32_t batch)
{
    dsxFatal(dsx_clear_unit(pUnit, pBias1, pBias2, pBias3, pBias4, 4, stride, batch), "kClearQuadSourceUnit");
}

void kCalculateSparseZ(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pWeight, uint64_t* pSparseStart, uint64_t* pSparseEnd,
                       uint32_t* pSparseIndex, NNFloat* pDataWeight, NNFloat* pUnit, NNFloat beta)
{
    uint32_t attr = DSX_ATTR_SPARSE | DSX_ATTR_BOOLEAN | (pDataWeight ? DSX_ATTR_WEIGHTED : 0);
    dsxFatal(dsx_sparse_z(attr, DSX_T_FLOAT, position, batch, stride, pWeight, NULL, pSparseStart, pSparseEnd, pSparseIndex, pDataWeight,
                          NULL, pUnit, beta), "kCalculateSparseZ");
}

void kCalculateIndexedSparseZ(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pWeight, uint32_t* pIndex, uint64_t* pSparseStart,
                              uint64_t* pSparseEnd, uint32_t* pSparseIndex, NNFloat* pDataWeight, NNFloat* pUnit, NNFloat beta)
{
    uint32_t attr = DSX_ATTR_SPARSE | DSX_ATTR_BOOLEAN | DSX_ATTR_INDEXED | (pDataWeight ? DSX_ATTR_WEIGHTED : 0);
    dsxFatal(dsx_sparse_z(attr, DSX_T_FLOAT, position, batch, stride, pWeight, pIndex, pSparseStart, pSparseEnd, pSparseIndex, pDataWeight,
                          NULL, pUnit, beta), "kCalculateIndexedSparseZ");
}

template <typename T>
void kCalculateSparseAnalogZ(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pWeight, uint64_t* pSparseStart, uint64_t* pSparseEnd,
                             uint32_t* pSparseIndex, NNFloat* pDataWeight, T* pSparseData, NNFloat* pUnit, NNFloat beta)
{
    uint32_t attr = DSX_ATTR_SPARSE | (pDataWeight ? DSX_ATTR_WEIGHTED : 0);
    dsxFatal(dsx_sparse_z(attr, (uint32_t)NNDataSetEnums::getDataType<T>(), position, batch, stride, pWeight, NULL, pSparseStart, pSparseEnd,
                          pSparseIndex, pDataWeight, pSparseData, pUnit, beta), "kCalculateSparseAnalogZ");
}

template <typename T>
void kCalculateIndexedSparseAnalogZ(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pWeight, uint32_t* pIndex,
                                    uint64_t* pSparseStart, uint64_t* pSparseEnd, uint32_t* pSparseIndex, NNFloat* pDataWeight, T* pSparseData,
                                    NNFloat* pUnit, NNFloat beta)
{
    uint32_t attr = DSX_ATTR_SPARSE | DSX_ATTR_INDEXED | (pDataWeight ? DSX_ATTR_WEIGHTED : 0);
    dsxFatal(dsx_sparse_z(attr, (uint32_t)NNDataSetEnums::getDataType<T>(), position, batch, stride, pWeight, pIndex, pSparseStart,
                          pSparseEnd, pSparseIndex, pDataWeight, pSparseData, pUnit, beta), "kCalculateIndexedSparseAnalogZ");
}

#define DSX_INSTANTIATE(T)                                                                                                              \
    template void kCalculateSparseAnalogZ<T>(uint32_t, uint32_t, uint32_t, NNFloat*, uint64_t*, uint64_t*, uint32_t*, NNFloat*, T*,      \
                                             NNFloat*, NNFloat);                                                                         \
    template void kCalculateIndexedSparseAnalogZ<T>(uint32_t, uint32_t, uint32_t, NNFloat*, uint32_t*, uint64_t*, uint64_t*, uint32_t*,  \
                                                    NNFloat*, T*, NNFloat*, NNFloat);
DSX_INSTANTIATE(uint32_t)
DSX_INSTANTIATE(int32_t)
DSX_INSTANTIATE(int64_t)
DSX_INSTANTIATE(uint64_t)
DSX_INSTANTIATE(float)
DSX_INSTANTIATE(double)
DSX_INSTANTIATE(char)
DSX_INSTANTIATE(unsigned char)
#undef DSX_INSTANTIATE

static void activation1D(NNFloat* pData, uint64_t size, uint32_t act, NNFloat slope, NNFloat alpha, NNFloat lambda, const char* what)
{
    dsx_act_params p = {slope, alpha, lambda};
    // elementwise: any factorisation of size into (batch, stride) works
    uint64_t stride = size, batch = 1;
    while (stride > 0x7fffffffull && (stride % 2) == 0) {
        stride /= 2;
        batch *= 2;
    }
    dsxFatal(dsx_activation(pData, (uint32_t)batch, (uint32_t)stride, act, &p), what);
}

void kCalculateSigmoidActivation(NNFloat* pData, uint64_t size) { activation1D(pData, size, DSX_ACT_SIGMOID, 0, 0, 0, "kCalculateSigmoidActivation"); }
void kCalculateTanhActivation(NNFloat* pData, uint64_t size) { activation1D(pData, size, DSX_ACT_TANH, 0, 0, 0, "kCalculateTanhActivation"); }
void kCalculateRELUActivation(NNFloat* pData, uint64_t size) { activation1D(pData, size, DSX_ACT_RELU, 0, 0, 0, "kCalculateRELUActivation"); }
void kCalculateLRELUActivation(NNFloat* pData, uint64_t size, NNFloat slope) { activation1D(pData, size, DSX_ACT_LRELU, slope, 0, 0, "kCalculateLRELUActivation"); }
void kCalculateELUActivation(NNFloat* pData, uint64_t size, NNFloat alpha) { activation1D(pData, size, DSX_ACT_ELU, 0, alpha, 0, "kCalculateELUActivation"); }
void kCalculateSELUActivation(NNFloat* pData, uint64_t size, NNFloat alpha, NNFloat lambda)
{
    activation1D(pData, size, DSX_ACT_SELU, 0, alpha, lambda, "kCalculateSELUActivation");
}
void kCalculateSoftMaxActivation(NNFloat* pData, uint32_t batch, uint32_t stride)
{
    dsxFatal(dsx_activation(pData, batch, stride, DSX_ACT_SOFTMAX, NULL), "kCalculateSoftMaxActivation");
}

void kAddBuffers(NNFloat* pDest, NNFloat* pSrc, uint64_t size) { dsxFatal(dsx_add_buffers(pDest, pSrc, size), "kAddBuffers"); }

void kCalculateTopK(NNFloat* pOutputKey, NNFloat* pKey, uint32_t* pValue, uint32_t batch, uint32_t width, uint32_t k)
{
    dsxFatal(dsx_topk(pOutputKey, pKey, pValue, batch, width, k), "kCalculateTopK");
}
void kCalculateTopK(NNFloat* pOutputKey, NNFloat* pOutputValue, NNFloat* pKey, NNFloat* pValue, uint32_t batch, uint32_t width, uint32_t k)
{
    dsxFatal(dsx_topk_kv_f32(pOutputKey, pOutputValue, pKey, pValue, batch, width, k), "kCalculateTopK");
}
void kCalculateTopK(NNFloat* pOutputKey, uint32_t* pOutputValue, NNFloat* pKey, uint32_t* pValue, uint32_t batch, uint32_t width, uint32_t k)
{
    dsxFatal(dsx_topk_kv_u32(pOutputKey, pOutputValue, pKey, pValue, batch, width, k), "kCalculateTopK");
}
