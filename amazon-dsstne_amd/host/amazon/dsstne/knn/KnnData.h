// KnnData.h — device-resident item table and result buffers of the exact KNN search (reference: knn/KnnData.h:33-140).
// One GPU: numGpus must be 1.  The item table is stored column-major [rowsPadded x D] as the reference builds it.
#ifndef DSSTNE_AMD_KNN_KNNDATA_H
#define DSSTNE_AMD_KNN_KNNDATA_H

#include <cstdint>
#include <map>
#include <string>
#include <vector>

#include "DataReader.h"

namespace astdl {
namespace knn {

// FP32 and FP16 as in the reference (knn/KnnData.h).  FP32Split ("fp32-split") has no counterpart there: fp32 storage whose
// inner products are formed from bf16 matrix instructions (dsx_knn_search_split): fp32-accurate scores, not bit-identical to
// FP32's, about 1.5 times as fast; the table is kept as bf16 planes, 1.5 times its fp32 size.
enum class DataType { FP32 = 0, FP16 = 1, FP32Split = 2 };

std::string getDataTypeString(DataType dataType);
DataType getDataTypeFromString(const std::string& dataTypeLiteral);

enum class MemoryType { Host = 1, Device = 2 };

struct Matrix {
    void* data;
    uint32_t numRows;
    int numColumns;
    size_t elementSize;
    MemoryType memoryType;

    Matrix();
    Matrix(void* data, uint32_t numRows, int numColumns, size_t elementSize, MemoryType memoryType);
    size_t getSizeInBytes();
    size_t getLength();
};

Matrix loadDataOnHost(DataReader* dataReader);

struct KnnData {
    const int numGpus;
    const int batchSize;
    const int maxK;

    std::vector<Matrix> dCollectionPartitions;   // column major
    std::vector<Matrix> dInputBatches;
    std::vector<Matrix> dResultScores;
    std::vector<Matrix> dResultIndexes;
    std::vector<Matrix> hResultScores;
    std::vector<Matrix> hResultIndexes;
    std::vector<std::vector<std::string>> hKeys;
    std::vector<Matrix> dWorkspaces;             // score blocks + partial lists of the search (instead of a full product matrix)
    std::vector<uint32_t> collectionRowsPadded;  // pad rows per device (rows are padded to a multiple of 8)
    std::vector<float> elapsedSgemm;             // milliseconds of the last search, per device
    std::vector<float> elapsedTopK;
    const DataType dataType;

    KnnData(int numGpus, int batchSize, int maxK, DataType dataType);
    void load(int device, DataReader* dataReader);
    void load(const std::map<int, DataReader*>& deviceToData);
    void load(const std::map<int, std::string>& deviceToFile, char keyValDelim, char vecDelim);
    int getFeatureSize() const;
    ~KnnData();
};

Matrix allocateMatrixOnHost(uint32_t numRows, int numColumns, size_t elementSize);
Matrix allocateMatrixOnDevice(uint32_t numRows, int numColumns, size_t elementSize);
void freeMatrix(const Matrix& matrix);

}  // namespace knn
}  // namespace astdl

#endif
