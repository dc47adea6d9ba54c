// KnnExactGpu.h — exact k-nearest-neighbour search by dot product (reference: knn/KnnExactGpu.h:27-69).
#ifndef DSSTNE_AMD_KNN_KNNEXACTGPU_H
#define DSSTNE_AMD_KNN_KNNEXACTGPU_H

#include <string>
#include <vector>

#include "KnnData.h"

namespace astdl {
namespace knn {

class Knn {
public:
    virtual void search(int k, const float* inputs, std::string* keys, float* scores) = 0;
    virtual ~Knn() {}

protected:
    KnnData* data;
    Knn(KnnData* data);
};

class KnnExactGpu : public Knn {
public:
    KnnExactGpu(KnnData* data);
    // inputs: [size][featureSize] row-major queries; keys / scores: [size][k], best first.
    void search(int k, const float* inputs, int size, std::string* keys, float* scores);
    void search(int k, const float* inputs, std::string* keys, float* scores) override { search(k, inputs, data->batchSize, keys, scores); }
};

// k-way merge of per-device result lists (each [batchSize][width], descending); ties go to the lower device id.
void mergeKnn(int k, int batchSize, int width, int numGpus, const std::vector<float*>& allScores, const std::vector<uint32_t*>& allIndexes,
              const std::vector<std::vector<std::string>>& allKeys, float* scores, std::string* keys);

}  // namespace knn
}  // namespace astdl

#endif
