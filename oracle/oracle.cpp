// oracle.cpp — TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// CPU restatement of the arithmetic of DSSTNE's sparse-recommendation inference path
// (sparse input -> fully connected stack -> filtered top-K, and the KNN dot-product + top-K module).
// DSSTNE itself has no CPU forward pass, so this file restates what its CUDA kernels compute, in
// scalar fp32 C++ with OpenMP over batch rows.  Only tests, the smoke check and the benchmark's
// cpu_baseline leg may load this library, and only as the checker / the reported CPU baseline.
// The product path (the HIP library) never links or calls it.
//
// Each function names the reference file:line it follows (paths relative to the reference root,
// "engine/" = src/amazon/dsstne/engine/, "utils/" = src/amazon/dsstne/utils/, "knn/" = src/amazon/dsstne/knn/).
//
// Pinning status (what independent evidence each function is checked against in tests/):
//   orc_topk            reference's own CPU routine topKsort (compiled from utils/Utils.cpp into oracle/_ref),
//                       shapes of tst/gputests/TestSort.cpp:208-211, brute force, invariants.
//   orc_sparse_z        dense identity X.W in fp64 (numpy), empty-row / single-nnz / duplicate-index special
//                       cases, indexed = row permutation, 8-bit scalings read from engine/kernels.cu:923,998.
//   orc_sgemm, orc_activation, orc_clear_unit, orc_forward
//                       textbook fp64 GEMM + closed-form activations (numpy / torch-CPU as independent code).
//                       The reference's GEMM lives in cuBLAS (closed source): summation order is PARITY UNPINNED
//                       and covered by the 1e-4 relative tolerance.
//   orc_apply_filter    definition in utils/Filters.cpp:49-67 + invariants (no filtered index in top-K).
//   orc_knn_search      fp64 Q.I^T + full sort (numpy), self-query invariant.
//   orc_softmax         closed form; the reference's 2^30 fixed-point accumulation is PARITY UNPINNED.
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <limits>
#include <numeric>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

// engine/NNTypes.h:49
constexpr float kMaxValue = 999999999999999.0f;

// engine/NNEnum.h:9-19 (dataset attribute bits)
enum : uint32_t { kSparse = 1, kBoolean = 2, kIndexed = 64, kWeighted = 128 };
// engine/NNEnum.h:35-47
enum : uint32_t { tUInt = 0, tInt = 1, tLLInt = 2, tULLInt = 3, tFloat = 4, tDouble = 5, tRGB8 = 6, tRGB16 = 7, tUChar = 8, tChar = 9 };
// engine/NNTypes.h:91-105 (Activation ordinals)
enum : uint32_t { aSigmoid = 0, aTanh = 1, aRELU = 2, aLinear = 3, aParametricRELU = 4, aSoftPlus = 5, aSoftSign = 6, aSoftMax = 7,
                  aRELUMax = 8, aLinearMax = 9, aELU = 10, aLRELU = 11, aSELU = 12 };

// Row resolution: engine/kernels.cu:670 (position + blockIdx.x), :750 (pIndex[...] when the dataset is Indexed).
inline uint32_t resolve_row(uint32_t position, uint32_t b, const uint32_t* index)
{
    uint32_t r = position + b;
    return index ? index[r] : r;
}

// engine/kernels.cu:837-893: generic analog kernel keeps "w * data" in a __shared__ T, i.e. the product is
// converted back to T before use; engine/kernels.cu:923,998: the uchar/char specialisations keep a float
// and scale the raw byte by 1/256.
template <typename T> struct AnalogValue {
    static inline T make(float w, T v) { return (T)(w * v); }
};
template <> struct AnalogValue<unsigned char> {
    static inline float make(float w, unsigned char v) { return w * ((float)v * (float)(1.0 / 256.0)); }
};
template <> struct AnalogValue<char> {
    static inline float make(float w, char v) { return w * ((float)v * (float)(1.0 / 256.0)); }
};

// unit += W * value with the multiply-add contracted, as nvcc does for engine/kernels.cu:706 / :868.
inline float madd(float a, float b, float c) { return std::fmaf(a, b, c); }
inline float madd(float a, double b, float c) { return (float)std::fma((double)a, b, (double)c); }
template <typename V> inline float madd(float a, V b, float c) { return std::fmaf(a, (float)b, c); }

template <typename T>
void sparse_analog_z(uint32_t position, uint32_t batch, uint32_t stride, const float* W, const uint32_t* index,
                     const uint64_t* start, const uint64_t* end, const uint32_t* sidx, const float* dw, const T* sdata,
                     float* unit, float beta)
{
#pragma omp parallel for schedule(dynamic, 4)
    for (int64_t b = 0; b < (int64_t)batch; b++) {
        uint32_t r = resolve_row(position, (uint32_t)b, index);
        uint64_t s = start[r], e = end[r];
        float w = dw ? dw[r] : 1.0f;
        float* u = unit + (uint64_t)b * stride;
        if (s >= e) continue;  // while (start < end) never entered: unit keeps its value, beta is not applied
        std::vector<float> acc(stride);
        for (uint32_t j = 0; j < stride; j++) acc[j] = (beta == 0.0f) ? 0.0f : beta * u[j];
        for (uint64_t t = s; t < e; t++) {
            auto v = AnalogValue<T>::make(w, sdata[t]);
            const float* wr = W + (uint64_t)sidx[t] * stride;
            for (uint32_t j = 0; j < stride; j++) acc[j] = madd(wr[j], v, acc[j]);
        }
        std::memcpy(u, acc.data(), sizeof(float) * stride);
    }
}

void sparse_boolean_z(uint32_t position, uint32_t batch, uint32_t stride, const float* W, const uint32_t* index,
                      const uint64_t* start, const uint64_t* end, const uint32_t* sidx, const float* dw, float* unit, float beta)
{
#pragma omp parallel for schedule(dynamic, 4)
    for (int64_t b = 0; b < (int64_t)batch; b++) {
        uint32_t r = resolve_row(position, (uint32_t)b, index);
        uint64_t s = start[r], e = end[r];
        float w = dw ? dw[r] : 1.0f;
        float* u = unit + (uint64_t)b * stride;
        if (s >= e) continue;
        std::vector<float> acc(stride);
        for (uint32_t j = 0; j < stride; j++) acc[j] = (beta == 0.0f) ? 0.0f : beta * u[j];
        for (uint64_t t = s; t < e; t++) {
            const float* wr = W + (uint64_t)sidx[t] * stride;
            for (uint32_t j = 0; j < stride; j++) acc[j] = std::fmaf(w, wr[j], acc[j]);   // engine/kernels.cu:706
        }
        std::memcpy(u, acc.data(), sizeof(float) * stride);
    }
}

struct Cand {
    float key;
    uint32_t idx;
};
// Build contract for ordering: score descending, ties broken by the lower index.
inline bool cand_before(const Cand& a, const Cand& b)
{
    if (a.key > b.key) return true;
    if (a.key < b.key) return false;
    return a.idx < b.idx;
}

void topk_row(const float* in, uint32_t width, uint32_t k, float* keys, uint32_t* idx, std::vector<Cand>& tmp)
{
    tmp.resize(width);
    for (uint32_t j = 0; j < width; j++) tmp[j] = Cand{in[j] + 0.0f, j};
    uint32_t m = std::min(k, width);
    std::partial_sort(tmp.begin(), tmp.begin() + m, tmp.end(), cand_before);
    for (uint32_t j = 0; j < m; j++) {
        keys[j] = tmp[j].key;
        idx[j] = tmp[j].idx;
    }
    // engine/kernels.cu:3221-3224: unfilled slots hold key -MAX_VALUE and index 0
    for (uint32_t j = m; j < k; j++) {
        keys[j] = -kMaxValue;
        idx[j] = 0;
    }
}

inline float act1(float x, uint32_t act, float slope, float alpha, float lambda)
{
    switch (act) {
    case aSigmoid: return 1.0f / (1.0f + std::exp(-x));               // engine/kActivation.cu:53
    case aTanh: return std::tanh(x);                                   // :72
    case aRELU: return std::max(0.0f, x);                              // :88
    case aLRELU: return std::max(x, x * slope);                        // :105-106
    case aELU: return (x > 0.0f) ? x : alpha * (std::exp(x) - 1.0f);   // :124-125
    case aSELU: return (x > 0.0f) ? lambda * x : lambda * alpha * (std::exp(x) - 1.0f);   // :143-144
    default: return x;                                                 // Linear and the *Max kinds: identity here
    }
}

}  // namespace

extern "C" {

int orc_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

// kClearUnit / kClearDualSourceUnit / Triple / Quad — engine/kernels.cu:61-145.
// unit[b][j] = sum_i bias_i[j].  (The reference's Triple/Quad variants index bias 3 and 4 with the flat position
// instead of the column, an upstream defect at :114,:135; the column is used here.)  nbias == 0 -> zero fill
// (engine/NNLayer.cpp:1002-1039 uses cudaMemset for a layer with no incoming weight).
void orc_clear_unit(float* unit, const float* const* bias, uint32_t nbias, uint32_t stride, uint32_t batch)
{
#pragma omp parallel for
    for (int64_t b = 0; b < (int64_t)batch; b++) {
        float* u = unit + (uint64_t)b * stride;
        for (uint32_t j = 0; j < stride; j++) {
            float s = 0.0f;
            if (nbias > 0) {
                s = bias[0][j];
                for (uint32_t i = 1; i < nbias; i++) s += bias[i][j];
            }
            u[j] = s;
        }
    }
}

// kCalculateSparseZ / kCalculateIndexedSparseZ / kCalculateSparseAnalogZ<T> / kCalculateIndexedSparseAnalogZ<T>
// — engine/kernels.cu:662-1299, dispatch engine/NNTypes.h:527-545.
// attributes: NNDataSetEnums::Attributes bits (Boolean selects the value-free kernel; Indexed is implied by index != NULL).
// data_type: NNDataSetEnums::DataType of sparse_data (ignored when Boolean).
int orc_sparse_z(uint32_t attributes, uint32_t data_type, uint32_t position, uint32_t batch, uint32_t stride, const float* W,
                 const uint32_t* index, const uint64_t* start, const uint64_t* end, const uint32_t* sparse_index,
                 const float* data_weight, const void* sparse_data, float* unit, float beta)
{
    if (!(attributes & kIndexed)) index = nullptr;
    if (!(attributes & kWeighted)) data_weight = nullptr;
    if (attributes & kBoolean) {
        sparse_boolean_z(position, batch, stride, W, index, start, end, sparse_index, data_weight, unit, beta);
        return 0;
    }
#define ORC_CASE(tag, T)                                                                                                             \
    case tag:                                                                                                                        \
        sparse_analog_z<T>(position, batch, stride, W, index, start, end, sparse_index, data_weight, (const T*)sparse_data, unit, beta); \
        return 0;
    switch (data_type) {
        ORC_CASE(tUInt, uint32_t)
        ORC_CASE(tInt, int32_t)
        ORC_CASE(tLLInt, int64_t)
        ORC_CASE(tULLInt, uint64_t)
        ORC_CASE(tFloat, float)
        ORC_CASE(tDouble, double)
        ORC_CASE(tUChar, unsigned char)
        ORC_CASE(tChar, char)
    default: return -1;
    }
#undef ORC_CASE
}

// kLoadSparseInputUnit / Indexed / Analog / IndexedAnalog — engine/kernels.cu:147-286.
// Row is zero-filled, then unit[b][sparse_index[t]] = w (Boolean) or w * value (analog, engine/kernels.cu:215-234; this
// loader has no 8-bit specialisation, so bytes are NOT rescaled here, unlike the sparse-Z kernels).  Later duplicates
// overwrite earlier ones.
int orc_load_sparse_input_unit(uint32_t attributes, uint32_t data_type, uint32_t position, uint32_t batch, uint32_t stride,
                               float* unit, const uint32_t* index, const uint64_t* start, const uint64_t* end,
                               const uint32_t* sparse_index, const float* data_weight, const void* sparse_data)
{
    if (!(attributes & kIndexed)) index = nullptr;
    if (!(attributes & kWeighted)) data_weight = nullptr;
    for (uint32_t b = 0; b < batch; b++) {
        uint32_t r = resolve_row(position, b, index);
        float w = data_weight ? data_weight[r] : 1.0f;
        float* u = unit + (uint64_t)b * stride;
        std::memset(u, 0, sizeof(float) * stride);
        for (uint64_t t = start[r]; t < end[r]; t++) {
            float v = w;
            if (!(attributes & kBoolean)) {
                switch (data_type) {
                case tUInt: v = w * ((const uint32_t*)sparse_data)[t]; break;
                case tInt: v = w * ((const int32_t*)sparse_data)[t]; break;
                case tLLInt: v = w * ((const int64_t*)sparse_data)[t]; break;
                case tULLInt: v = w * ((const uint64_t*)sparse_data)[t]; break;
                case tFloat: v = w * ((const float*)sparse_data)[t]; break;
                case tDouble: v = (float)(w * ((const double*)sparse_data)[t]); break;
                case tUChar: v = w * ((const unsigned char*)sparse_data)[t]; break;
                case tChar: v = w * ((const char*)sparse_data)[t]; break;
                default: return -1;
                }
            }
            u[sparse_index[t]] = v;
        }
    }
    return 0;
}

// kLoadInputUnit<T> / kLoadIndexedInputUnit<T> — engine/kernels.cu:439-562: dense row copy with conversion;
// uchar -> x/256 - 0.5 (:463), char -> x/128 (:476).
int orc_load_input_unit(uint32_t data_type, uint32_t position, uint32_t batch, uint32_t stride, float* unit,
                        const uint32_t* index, const void* data)
{
    for (uint32_t b = 0; b < batch; b++) {
        uint32_t r = resolve_row(position, b, index);
        float* u = unit + (uint64_t)b * stride;
        uint64_t so = (uint64_t)r * stride;
        for (uint32_t j = 0; j < stride; j++) {
            switch (data_type) {
            case tUInt: u[j] = (float)((const uint32_t*)data)[so + j]; break;
            case tInt: u[j] = (float)((const int32_t*)data)[so + j]; break;
            case tLLInt: u[j] = (float)((const int64_t*)data)[so + j]; break;
            case tULLInt: u[j] = (float)((const uint64_t*)data)[so + j]; break;
            case tFloat: u[j] = ((const float*)data)[so + j]; break;
            case tDouble: u[j] = (float)((const double*)data)[so + j]; break;
            case tUChar: u[j] = (float)((const unsigned char*)data)[so + j] * (float)(1.0 / 256.0) - 0.5f; break;
            case tChar: u[j] = (float)((const char*)data)[so + j] * (float)(1.0 / 128.0); break;
            default: return -1;
            }
        }
    }
    return 0;
}

// Forward GEMM of a fully connected layer: Z[B x n] += X[B x k] . W[k x n] (beta = 1 over the bias-initialised Z),
// engine/NNLayer.cpp:1056-1096.  Loop nest of the reference's only scalar GEMM, verifySGEMM
// (engine/GpuTypes.cpp:538-550): one output at a time, k innermost, fp32 accumulator.
// transposed != 0: W is held as [n x k] (shared transposed weights, engine/NNLayer.cpp:1065-1072).
void orc_sgemm(const float* X, const float* W, float* Z, uint32_t B, uint32_t k, uint32_t n, int transposed)
{
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < (int64_t)B; b++) {
        const float* x = X + (uint64_t)b * k;
        float* z = Z + (uint64_t)b * n;
        if (!transposed) {
            // k-outer / n-inner walks W rows contiguously; per output the additions happen in the same k order
            // as the k-innermost nest, so the result is identical.
            std::vector<float> acc(n, 0.0f);
            for (uint32_t kk = 0; kk < k; kk++) {
                float xv = x[kk];
                const float* wr = W + (uint64_t)kk * n;
                for (uint32_t j = 0; j < n; j++) acc[j] += xv * wr[j];
            }
            for (uint32_t j = 0; j < n; j++) z[j] += acc[j];
        } else {
            for (uint32_t j = 0; j < n; j++) {
                const float* wr = W + (uint64_t)j * k;
                float s = 0.0f;
                for (uint32_t kk = 0; kk < k; kk++) s += x[kk] * wr[kk];
                z[j] += s;
            }
        }
    }
}

// kAddBuffers — engine/kernels.cu:4763-4781 (skip connections, engine/NNLayer.cpp:1099-1103)
void orc_add_buffers(float* dst, const float* src, uint64_t size)
{
    for (uint64_t i = 0; i < size; i++) dst[i] += src[i];
}

// kCalculate{Sigmoid,Tanh,RELU,LRELU,ELU,SELU}Activation — engine/kActivation.cu:46-153, elementwise in place.
void orc_activation(float* z, uint64_t size, uint32_t act, float slope, float alpha, float lambda)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)size; i++) z[i] = act1(z[i], act, slope, alpha, lambda);
}

// kCalculateSoftMaxActivation — engine/kActivation.cu:155-236: subtract the row maximum, exponentiate,
// a = min(1, exp * (1/sum)).  (The reference accumulates the sum in 2^30 fixed point; a float sum is used here.)
void orc_softmax(float* z, uint32_t batch, uint32_t stride)
{
#pragma omp parallel for
    for (int64_t b = 0; b < (int64_t)batch; b++) {
        float* r = z + (uint64_t)b * stride;
        float m = -std::numeric_limits<float>::infinity();
        for (uint32_t j = 0; j < stride; j++) m = std::max(m, r[j]);
        double s = 0.0;
        for (uint32_t j = 0; j < stride; j++) s += std::exp(r[j] - m);
        float inv = (float)(1.0 / s);
        for (uint32_t j = 0; j < stride; j++) r[j] = std::min(1.0f, std::exp(r[j] - m) * inv);
    }
}

// kCalculateTopK(pOutput, pKey, pValue, batch, width, k) — engine/kernels.cu:3202-3989.
// Row pitch equals width.  Keys descending; order among equal keys is (by this build's contract) lower index first.
void orc_topk(const float* in, uint32_t batch, uint32_t width, uint32_t k, float* keys, uint32_t* idx)
{
#pragma omp parallel
    {
        std::vector<Cand> tmp;
#pragma omp for schedule(dynamic, 4)
        for (int64_t b = 0; b < (int64_t)batch; b++)
            topk_row(in + (uint64_t)b * width, width, k, keys + (uint64_t)b * k, idx + (uint64_t)b * k, tmp);
    }
}

// KNN variant — knn/topk.cu:29-229: row pitch `width`, only the first width - width_padding columns are candidates.
void orc_knn_topk(const float* in, uint32_t batch, uint32_t width, uint32_t width_padding, uint32_t k, float* keys, uint32_t* idx)
{
#pragma omp parallel
    {
        std::vector<Cand> tmp;
#pragma omp for schedule(dynamic, 4)
        for (int64_t b = 0; b < (int64_t)batch; b++)
            topk_row(in + (uint64_t)b * width, width - width_padding, k, keys + (uint64_t)b * k, idx + (uint64_t)b * k, tmp);
    }
}

// Key/value variants — engine/kernels.cu:3992-4385: top-k of (key, value) pairs, keys descending.  Ties are broken by
// the lower source column (build contract).  value_is_u32 selects the uint32 payload overload.
void orc_topk_kv(const float* in_key, const void* in_val, uint32_t batch, uint32_t width, uint32_t k, float* keys, void* vals,
                 int value_is_u32)
{
#pragma omp parallel
    {
        std::vector<Cand> tmp;
        std::vector<float> kk(k);
        std::vector<uint32_t> ii(k);
#pragma omp for schedule(dynamic, 4)
        for (int64_t b = 0; b < (int64_t)batch; b++) {
            topk_row(in_key + (uint64_t)b * width, width, k, kk.data(), ii.data(), tmp);
            uint32_t m = std::min(k, width);
            for (uint32_t j = 0; j < k; j++) {
                keys[(uint64_t)b * k + j] = kk[j];
                if (value_is_u32)
                    ((uint32_t*)vals)[(uint64_t)b * k + j] = (j < m) ? ((const uint32_t*)in_val)[(uint64_t)b * width + ii[j]] : 0u;
                else
                    ((float*)vals)[(uint64_t)b * k + j] = (j < m) ? ((const float*)in_val)[(uint64_t)b * width + ii[j]] : 0.0f;
            }
        }
    }
}

// AbstractFilter::updateRecords(xArray, xFilter, offset, width) — utils/Filters.cpp:49-67, driven per sample by
// utils/NNRecsGenerator.cpp:138-145: score[idx - offset] *= value for every (idx, value) of the sample's filter with
// idx in [offset, offset + width).  The filter of batch row b is CSR row resolve_row(position, b, index); mul == NULL
// means every value is 0.0f (a feature listed without a value, utils/Filters.cpp:108-121).  An index listed twice is
// applied once (the reference keeps the filter in a map keyed by index).
void orc_apply_filter(float* scores, uint32_t batch, uint32_t width, uint32_t offset, uint32_t position, const uint32_t* index,
                      const uint64_t* fstart, const uint64_t* fend, const uint32_t* fidx, const float* fmul)
{
#pragma omp parallel
    {
        std::vector<uint8_t> seen(width);
#pragma omp for schedule(dynamic, 4)
        for (int64_t b = 0; b < (int64_t)batch; b++) {
            uint32_t r = resolve_row(position, (uint32_t)b, index);
            float* s = scores + (uint64_t)b * width;
            for (uint64_t t = fstart[r]; t < fend[r]; t++) {
                uint32_t i = fidx[t];
                if (i < offset || i >= offset + width) continue;
                if (seen[i - offset]) continue;
                seen[i - offset] = 1;
                float v = fmul ? fmul[t] : 0.0f;
                s[i - offset] = v * s[i - offset];
            }
            for (uint64_t t = fstart[r]; t < fend[r]; t++) {
                uint32_t i = fidx[t];
                if (i >= offset && i < offset + width) seen[i - offset] = 0;
            }
        }
    }
}

// Filtered recommendations: utils/NNRecsGenerator.cpp:132-150 — filter multiply on a copy of the output rows, then top-k.
void orc_topk_filtered(const float* in, uint32_t batch, uint32_t width, uint32_t k, uint32_t position, const uint32_t* index,
                       const uint64_t* fstart, const uint64_t* fend, const uint32_t* fidx, const float* fmul, float* keys,
                       uint32_t* idx)
{
    std::vector<float> tmp((uint64_t)batch * width);
    std::memcpy(tmp.data(), in, sizeof(float) * (uint64_t)batch * width);
    orc_apply_filter(tmp.data(), batch, width, 0, position, index, fstart, fend, fidx, fmul);
    orc_topk(tmp.data(), batch, width, k, keys, idx);
}

// KnnExactGpu::search on one device — knn/KnnExactGpu.cu:43-159 with knn/KnnData.cpp:180-240 layout:
// items column-major [rows_padded x D] (items[d * rows_padded + m]), queries row-major [Q x D];
// scores[q][m] = sum_d items[m,d] * queries[q,d]; top-k over the first rows_padded - padding columns.
void orc_knn_search(const float* items, uint32_t rows_padded, uint32_t padding, uint32_t D, const float* queries, uint32_t Q,
                    uint32_t k, float* scores, uint32_t* idx)
{
    uint32_t M = rows_padded - padding;
#pragma omp parallel
    {
        std::vector<float> row(M);
        std::vector<Cand> tmp;
#pragma omp for schedule(dynamic, 1)
        for (int64_t q = 0; q < (int64_t)Q; q++) {
            std::fill(row.begin(), row.end(), 0.0f);
            for (uint32_t d = 0; d < D; d++) {
                float qv = queries[(uint64_t)q * D + d];
                const float* col = items + (uint64_t)d * rows_padded;
                for (uint32_t m = 0; m < M; m++) row[m] += qv * col[m];
            }
            topk_row(row.data(), M, k, scores + (uint64_t)q * k, idx + (uint64_t)q * k, tmp);
        }
    }
}

// mergeKnn — knn/KnnExactGpu.cu:161-198: k-way merge of per-device descending lists (pitch `width`),
// strict '<' so the lowest device id wins ties.  Emits indexes (the reference maps them to string keys).
void orc_merge_knn(uint32_t k, uint32_t batch, uint32_t width, uint32_t ndev, const float* const* all_scores,
                   const uint32_t* const* all_idx, float* scores, uint32_t* idx, uint32_t* dev)
{
    for (uint32_t i = 0; i < batch; i++) {
        std::vector<uint32_t> pos(ndev, i * width);
        for (uint32_t c = 0; c < k; c++) {
            uint32_t best = 0;
            float mv = all_scores[0][pos[0]];
            for (uint32_t d = 0; d < ndev; d++)
                if (mv < all_scores[d][pos[d]]) {
                    mv = all_scores[d][pos[d]];
                    best = d;
                }
            scores[(uint64_t)i * k + c] = mv;
            idx[(uint64_t)i * k + c] = all_idx[best][pos[best]];
            if (dev) dev[(uint64_t)i * k + c] = best;
            pos[best]++;
        }
    }
}

// Whole forward pass for a chain network (NNNetwork::PredictBatch -> NNLayer::ForwardPropagateFullyConnected,
// engine/NNNetwork.cpp:1376-1429, engine/NNLayer.cpp:994-1168, single process) followed by the filtered top-K of
// utils/NNRecsGenerator.cpp:132-150 with the sample's own inputs as its filter.
//   layer 0: sparse input (fast-sparse path): z = bias; z += sparse Z; activation
//   layer l > 0: z = bias; z += a_{l-1} . W_l; activation
// widths[0] = input width, widths[1..nlayers] = layer widths; W[l] is [widths[l] x widths[l+1]] row-major.
// unit_out (optional) receives the last layer's activations [batch x widths[nlayers]].
// Returns elapsed seconds of the computation (steady clock), so the benchmark can report a CPU baseline.
double orc_forward(uint32_t nlayers, const uint32_t* widths, const float* const* W, const float* const* bias, const uint32_t* acts,
                   uint32_t attributes, uint32_t data_type, uint32_t position, uint32_t batch, const uint32_t* index,
                   const uint64_t* start, const uint64_t* end, const uint32_t* sparse_index, const float* data_weight,
                   const void* sparse_data, uint32_t k, int filtered, float* unit_out, float* keys, uint32_t* idx)
{
    auto t0 = std::chrono::steady_clock::now();
    std::vector<float> cur, nxt;
    for (uint32_t l = 0; l < nlayers; l++) {
        uint32_t n = widths[l + 1];
        nxt.assign((uint64_t)batch * n, 0.0f);
        const float* b1[1] = {bias[l]};
        orc_clear_unit(nxt.data(), b1, 1, n, batch);
        if (l == 0)
            orc_sparse_z(attributes, data_type, position, batch, n, W[0], index, start, end, sparse_index, data_weight, sparse_data,
                         nxt.data(), 1.0f);
        else
            orc_sgemm(cur.data(), W[l], nxt.data(), batch, widths[l], n, 0);
        if (acts[l] == aSoftMax)
            orc_softmax(nxt.data(), batch, n);
        else
            orc_activation(nxt.data(), (uint64_t)batch * n, acts[l], 0.01f, 1.0f, 1.0f);
        cur.swap(nxt);
    }
    uint32_t N = widths[nlayers];
    if (keys && idx) {
        if (filtered) {
            const uint32_t* ix = (attributes & kIndexed) ? index : nullptr;
            orc_apply_filter(cur.data(), batch, N, 0, position, ix, start, end, sparse_index, nullptr);
        }
        orc_topk(cur.data(), batch, N, k, keys, idx);
    }
    auto t1 = std::chrono::steady_clock::now();
    // note: with `filtered`, unit_out receives the post-filter scores only if requested after filtering; callers that
    // want the raw activations pass keys == NULL.
    if (unit_out) std::memcpy(unit_out, cur.data(), sizeof(float) * (uint64_t)batch * N);
    return std::chrono::duration<double>(t1 - t0).count();
}

}  // extern "C"
