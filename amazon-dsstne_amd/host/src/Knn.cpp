// Knn.cpp — host side of the exact KNN module (reference: knn/KnnData.cpp:108-367, knn/KnnExactGpu.cu:43-198,
// knn/DataReader.cpp).  The device part is one call, dsx_knn_search, which never stores the full score matrix.
#include <cstring>
#include <sstream>
#include <stdexcept>

#include "amazon/dsstne/knn/KnnExactGpu.h"
#include "amazon/dsstne/knn/topk.h"
#include "dsx.h"

void kCalculateTopK(NNFloat* pOutput, NNFloat* pKey, uint32_t* pValue, uint32_t batch, uint32_t width, uint32_t widthPadding, uint32_t k)
{
    int rc = dsx_knn_topk(pOutput, pKey, pValue, batch, width, widthPadding, k);
    if (rc != DSX_OK) {
        printf("Error: %s launching kernel kCalculateTopK\n", dsx_last_error());
        exit(-1);
    }
}

// ------------------------------------------------------------------------------------------------------------ DataReader

static void splitRow(const std::string& line, char kv, char vd, std::string* key, float* vector, int columns, int* counted)
{
    size_t p = line.find(kv);
    if (p == std::string::npos) throw std::invalid_argument("Malformed line. key-value delimiter not found: " + line);
    if (key) *key = line.substr(0, p);
    int n = 0;
    size_t at = p + 1;
    while (at <= line.size()) {
        size_t e = line.find(vd, at);
        if (e == std::string::npos) e = line.size();
        if (e > at) {
            if (vector && n < columns) vector[n] = std::stof(line.substr(at, e - at));
            n++;
        }
        at = e + 1;
    }
    if (counted) *counted = n;
}

TextFileDataReader::TextFileDataReader(const std::string& fileName, char keyValueDelimiter, char vectorDelimiter)
    : fileName(fileName), fileStream(fileName, std::ios_base::in), keyValueDelimiter(keyValueDelimiter), vectorDelimiter(vectorDelimiter)
{
    findDataDimensions(fileName, rows, columns, keyValueDelimiter, vectorDelimiter);
}

void TextFileDataReader::findDataDimensions(const std::string& fileName, uint32_t& rows, int& columns, char keyValueDelimiter, char vectorDelimiter)
{
    std::fstream fs(fileName, std::ios_base::in);
    if (!fs) throw std::runtime_error("Cannot open " + fileName);
    rows = 0;
    columns = 0;
    std::string line;
    while (std::getline(fs, line)) {
        if (line.empty()) continue;
        ++rows;
        if (columns == 0) splitRow(line, keyValueDelimiter, vectorDelimiter, nullptr, nullptr, 0, &columns);
    }
}

bool TextFileDataReader::readRow(std::string* key, float* vector)
{
    std::string line;
    while (std::getline(fileStream, line)) {
        if (line.empty()) continue;
        int n = 0;
        splitRow(line, keyValueDelimiter, vectorDelimiter, key, vector, columns, &n);
        if (n != columns) {
            std::stringstream msg;
            msg << "Malformed row in " << fileName << ": expected " << columns << " values, found " << n;
            throw std::invalid_argument(msg.str());
        }
        return true;
    }
    return false;
}

TextFileDataReader::~TextFileDataReader() { fileStream.close(); }

ArrayDataReader::ArrayDataReader(const float* data, uint32_t rows_, int columns_, const std::string* keys) : data(data), keys(keys), next(0)
{
    rows = rows_;
    columns = columns_;
}

bool ArrayDataReader::readRow(std::string* key, float* vector)
{
    if (next >= rows) return false;
    if (key) *key = keys ? keys[next] : std::to_string(next);
    memcpy(vector, data + (size_t)next * columns, sizeof(float) * columns);
    ++next;
    return true;
}

namespace astdl {
namespace knn {

static const uint32_t ROW_PADDING = 8;

static void check(int rc, const char* what)
{
    if (rc != DSX_OK) throw std::runtime_error(std::string(what) + ": " + dsx_last_error());
}

std::string getDataTypeString(DataType dataType)
{
    switch (dataType) {
    case DataType::FP32: return "fp32";
    case DataType::FP16: return "fp16";
    case DataType::FP32Split: return "fp32-split";
    default: return "unknown";
    }
}

DataType getDataTypeFromString(const std::string& s)
{
    if (s == "fp32") return DataType::FP32;
    if (s == "fp16") return DataType::FP16;
    if (s == "fp32-split") return DataType::FP32Split;
    throw std::invalid_argument("Unknown DataType " + s);
}

Matrix::Matrix() : data(nullptr), numRows(0), numColumns(0), elementSize(0), memoryType(MemoryType::Host) {}
Matrix::Matrix(void* data, uint32_t numRows, int numColumns, size_t elementSize, MemoryType memoryType)
    : data(data), numRows(numRows), numColumns(numColumns), elementSize(elementSize), memoryType(memoryType)
{
}
size_t Matrix::getSizeInBytes() { return (size_t)numRows * numColumns * elementSize; }
size_t Matrix::getLength() { return (size_t)numRows * numColumns; }

Matrix allocateMatrixOnHost(uint32_t numRows, int numColumns, size_t elementSize)
{
    void* data = calloc((size_t)numRows * numColumns, elementSize);   // zeroed, so pad rows of the item table hold 0, not garbage
    return Matrix(data, numRows, numColumns, elementSize, MemoryType::Host);
}

Matrix allocateMatrixOnDevice(uint32_t numRows, int numColumns, size_t elementSize)
{
    void* data = nullptr;
    check(dsx_malloc(&data, (size_t)numRows * numColumns * elementSize), "allocateMatrixOnDevice");
    return Matrix(data, numRows, numColumns, elementSize, MemoryType::Device);
}

void freeMatrix(const Matrix& matrix)
{
    if (matrix.data == nullptr) return;
    if (matrix.memoryType == MemoryType::Device) {
        if (dsx_is_initialized()) check(dsx_free(matrix.data), "freeMatrix");
    } else {
        free(matrix.data);
    }
}

Matrix loadDataOnHost(DataReader* dataReader)
{
    uint32_t rows = dataReader->getRows();
    int columns = dataReader->getColumns();
    Matrix matrix = allocateMatrixOnHost(rows, columns, sizeof(float));
    std::string ignored;
    for (uint32_t r = 0; r < rows && dataReader->readRow(&ignored, ((float*)matrix.data) + (size_t)r * columns); ++r) {
    }
    return matrix;
}

KnnData::KnnData(int numGpus, int batchSize, int maxK, DataType dataType)
    : numGpus(numGpus), batchSize(batchSize), maxK(maxK), dCollectionPartitions(numGpus), dInputBatches(numGpus), dResultScores(numGpus),
      dResultIndexes(numGpus), hResultScores(numGpus), hResultIndexes(numGpus), hKeys(numGpus), dWorkspaces(numGpus),
      collectionRowsPadded(numGpus), elapsedSgemm(numGpus), elapsedTopK(numGpus), dataType(dataType)
{
    if (numGpus != 1) {
        std::stringstream msg;
        msg << "This build searches on exactly one GPU (the whole item table lives in one device's HBM). Required " << numGpus;
        throw std::runtime_error(msg.str());
    }
    if (maxK < 1 || maxK > 256) throw std::invalid_argument("maxK must be in 1..256");
    check(dsx_init(0), "KnnData");
    fprintf(stderr, "INFO: Initializing KnnData with numGpus = %d, batchSize = %d, maxK = %d, dataType = %s\n", numGpus, batchSize, maxK,
            getDataTypeString(dataType).c_str());
}

int KnnData::getFeatureSize() const { return dCollectionPartitions[0].numColumns; }

void KnnData::load(int device, DataReader* dataReader)
{
    if (device != 0) throw std::runtime_error("KnnData::load: only device 0 exists in this build");
    const uint32_t actualRows = dataReader->getRows();
    const uint32_t rows = ((actualRows + (ROW_PADDING - 1)) / ROW_PADDING) * ROW_PADDING;
    const int columns = dataReader->getColumns();
    collectionRowsPadded[device] = rows - actualRows;

    Matrix hTmp = allocateMatrixOnHost(rows, columns, sizeof(float));
    float* hTmpData = (float*)hTmp.data;
    std::string key;
    std::vector<float> vec(columns);
    hKeys[device].clear();
    for (uint32_t rowNum = 0; rowNum < actualRows && dataReader->readRow(&key, vec.data()); ++rowNum) {
        hKeys[device].push_back(key);
        for (int j = 0; j < columns; ++j) hTmpData[(size_t)j * rows + rowNum] = vec[j];   // column major
    }
    freeMatrix(dCollectionPartitions[device]);
    freeMatrix(dInputBatches[device]);
    freeMatrix(dResultScores[device]);
    freeMatrix(dResultIndexes[device]);
    freeMatrix(hResultScores[device]);
    freeMatrix(hResultIndexes[device]);
    freeMatrix(dWorkspaces[device]);
    if (dataType == DataType::FP16) {
        // knn/KnnData.cpp:209-216: the table is kept as halves (round to nearest even); the fp32 copy only lives until it is
        // converted.  The fp16 table has this library's padded item-major layout, so its Matrix describes the logical shape
        // (rows x columns of 2-byte elements) over an allocation of dsx_knn_f16_table_bytes.
        Matrix dTmp = allocateMatrixOnDevice(rows, columns, sizeof(float));
        check(dsx_memcpy_h2d(dTmp.data, hTmpData, hTmp.getSizeInBytes()), "KnnData::load");
        void* table = nullptr;
        check(dsx_malloc(&table, dsx_knn_f16_table_bytes(rows, (uint32_t)columns)), "KnnData::load");
        dCollectionPartitions[device] = Matrix(table, rows, columns, 2, MemoryType::Device);
        check(dsx_knn_f16_convert_items((const float*)dTmp.data, rows, rows - actualRows, (uint32_t)columns, table), "KnnData::load");
        check(dsx_sync(), "KnnData::load");
        freeMatrix(dTmp);
    } else if (dataType == DataType::FP32Split) {
        // the table as three planes of bf16 (dsx_fc_split of the column-major fp32 table, which only lives until then); its
        // Matrix describes the logical shape (rows x columns of 3 x 2 bytes) over an allocation of dsx_fc_split_bytes
        Matrix dTmp = allocateMatrixOnDevice(rows, columns, sizeof(float));
        check(dsx_memcpy_h2d(dTmp.data, hTmpData, hTmp.getSizeInBytes()), "KnnData::load");
        void* planes = nullptr;
        check(dsx_malloc(&planes, dsx_fc_split_bytes(rows, (uint32_t)columns)), "KnnData::load");
        dCollectionPartitions[device] = Matrix(planes, rows, columns, 6, MemoryType::Device);
        check(dsx_fc_split((const float*)dTmp.data, rows, 1, rows, (uint32_t)columns, planes), "KnnData::load");
        check(dsx_sync(), "KnnData::load");
        freeMatrix(dTmp);
    } else {
        dCollectionPartitions[device] = allocateMatrixOnDevice(rows, columns, sizeof(float));
        check(dsx_memcpy_h2d(dCollectionPartitions[device].data, hTmpData, hTmp.getSizeInBytes()), "KnnData::load");
    }
    freeMatrix(hTmp);
    dInputBatches[device] = allocateMatrixOnDevice(batchSize, columns, sizeof(float));
    dResultScores[device] = allocateMatrixOnDevice(batchSize, maxK, sizeof(float));
    dResultIndexes[device] = allocateMatrixOnDevice(batchSize, maxK, sizeof(uint32_t));
    hResultScores[device] = allocateMatrixOnHost(batchSize, maxK, sizeof(float));
    hResultIndexes[device] = allocateMatrixOnHost(batchSize, maxK, sizeof(uint32_t));
    const size_t ws = dataType == DataType::FP16        ? dsx_knn_workspace_bytes_f16(rows, columns, batchSize, maxK)
                      : dataType == DataType::FP32Split ? dsx_knn_workspace_bytes_split(rows, columns, batchSize, maxK)
                                                        : dsx_knn_workspace_bytes(rows, columns, batchSize, maxK);
    dWorkspaces[device] = allocateMatrixOnDevice(1, 1, ws);
    dsx_device_info info;
    check(dsx_get_device_info(&info), "KnnData::load");
    fprintf(stderr, "INFO: loaded %u (%u padded) rows and %d columns into device %d. Used: %zu MB, Free: %zu MB, Total: %zu MB\n", actualRows,
            rows, columns, device, (info.hbm_bytes - info.hbm_free_bytes) >> 20, info.hbm_free_bytes >> 20, info.hbm_bytes >> 20);
}

void KnnData::load(const std::map<int, DataReader*>& deviceToData)
{
    for (int device = 0; device < numGpus; device++) {
        auto it = deviceToData.find(device);
        if (it == deviceToData.end()) {
            std::stringstream msg;
            msg << "Data reader for device " << device << " not specified. Must specify readers for all " << numGpus << " devices";
            throw std::runtime_error(msg.str());
        }
        load(device, it->second);
    }
}

void KnnData::load(const std::map<int, std::string>& deviceToFile, char keyValDelim, char vecDelim)
{
    std::map<int, DataReader*> deviceToData;
    for (const auto& entry : deviceToFile) deviceToData.insert({entry.first, new TextFileDataReader(entry.second, keyValDelim, vecDelim)});
    try {
        load(deviceToData);
    } catch (...) {
        for (const auto& entry : deviceToData) delete entry.second;
        throw;
    }
    for (const auto& entry : deviceToData) delete entry.second;
}

KnnData::~KnnData()
{
    for (auto& m : dCollectionPartitions) freeMatrix(m);
    for (auto& m : dInputBatches) freeMatrix(m);
    for (auto& m : dResultScores) freeMatrix(m);
    for (auto& m : dResultIndexes) freeMatrix(m);
    for (auto& m : hResultScores) freeMatrix(m);
    for (auto& m : hResultIndexes) freeMatrix(m);
    for (auto& m : dWorkspaces) freeMatrix(m);
}

Knn::Knn(KnnData* data) : data(data) {}

KnnExactGpu::KnnExactGpu(KnnData* data) : Knn(data) {}

void KnnExactGpu::search(int k, const float* inputs, int size, std::string* keys, float* scores)
{
    const int maxK = data->maxK;
    if (k > maxK) {
        std::stringstream msg;
        msg << "k = " << k << " is > maxK = " << maxK;
        throw std::invalid_argument(msg.str());
    }
    if (size > data->batchSize) {
        // the reference builds this message and then forgets to throw it (knn/KnnExactGpu.cu:56-60); overrunning the query
        // buffer is never acceptable, so it is an error here
        std::stringstream msg;
        msg << "size = " << size << " is > batchSize = " << data->batchSize;
        throw std::invalid_argument(msg.str());
    }
    const int device = 0;
    Matrix& items = data->dCollectionPartitions[device];
    Matrix& dIn = data->dInputBatches[device];
    float* dScores = (float*)data->dResultScores[device].data;
    uint32_t* dIndexes = (uint32_t*)data->dResultIndexes[device].data;
    float* hScores = (float*)data->hResultScores[device].data;
    uint32_t* hIndexes = (uint32_t*)data->hResultIndexes[device].data;
    const int D = items.numColumns;

    check(dsx_memcpy_h2d(dIn.data, inputs, (size_t)size * D * sizeof(float)), "KnnExactGpu::search");
    float elapsed[2] = {0, 0};
    if (data->dataType == DataType::FP16)
        check(dsx_knn_search_f16(items.data, items.numRows, data->collectionRowsPadded[device], (uint32_t)D, (const float*)dIn.data,
                                 (uint32_t)size, (uint32_t)maxK, dScores, dIndexes, data->dWorkspaces[device].data,
                                 data->dWorkspaces[device].elementSize, elapsed),
              "KnnExactGpu::search");
    else if (data->dataType == DataType::FP32Split)
        check(dsx_knn_search_split(items.data, items.numRows, data->collectionRowsPadded[device], (uint32_t)D, (const float*)dIn.data,
                                   (uint32_t)size, (uint32_t)maxK, dScores, dIndexes, data->dWorkspaces[device].data,
                                   data->dWorkspaces[device].elementSize, elapsed),
              "KnnExactGpu::search");
    else
        check(dsx_knn_search((const float*)items.data, items.numRows, data->collectionRowsPadded[device], (uint32_t)D, (const float*)dIn.data,
                             (uint32_t)size, (uint32_t)maxK, dScores, dIndexes, data->dWorkspaces[device].data,
                             data->dWorkspaces[device].elementSize, elapsed),
              "KnnExactGpu::search");
    data->elapsedSgemm[device] = elapsed[0];
    data->elapsedTopK[device] = elapsed[1];
    check(dsx_memcpy_d2h(hScores, dScores, (size_t)size * maxK * sizeof(float)), "KnnExactGpu::search");
    check(dsx_memcpy_d2h(hIndexes, dIndexes, (size_t)size * maxK * sizeof(uint32_t)), "KnnExactGpu::search");

    std::vector<float*> allScores(1, hScores);
    std::vector<uint32_t*> allIndexes(1, hIndexes);
    mergeKnn(k, size, maxK, 1, allScores, allIndexes, data->hKeys, scores, keys);
}

void mergeKnn(int k, int batchSize, int width, int numGpus, const std::vector<float*>& allScores, const std::vector<uint32_t*>& allIndexes,
              const std::vector<std::vector<std::string>>& allKeys, float* scores, std::string* keys)
{
    std::vector<int> pos(numGpus);
    for (int i = 0; i < batchSize; ++i) {
        for (int n = 0; n < numGpus; n++) pos[n] = i * width;
        for (int col = 0; col < k; col++) {
            int best = 0;
            float maxVal = allScores[0][pos[0]];
            for (int dev = 1; dev < numGpus; dev++) {
                if (maxVal < allScores[dev][pos[dev]]) {   // strict: the lower device keeps ties
                    maxVal = allScores[dev][pos[dev]];
                    best = dev;
                }
            }
            const uint32_t idx = allIndexes[best][pos[best]];
            ++pos[best];
            scores[i * k + col] = maxVal;
            keys[i * k + col] = idx < allKeys[best].size() ? allKeys[best][idx] : std::string();
        }
    }
}

}  // namespace knn
}  // namespace astdl
