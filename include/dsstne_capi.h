/*
 * dsstne_capi.h — C ABI of libdsstne_amd.so over the C++ inference classes (NNNetwork, NNDataSet<T>, DsstneContext,
 * KnnExactGpu), shaped after the reference's own foreign-function surface: the JNI entry points of
 * java/src/main/native/com_amazon_dsstne_Dsstne.cpp (load :136-143, load_datasets :155-191, predict :272-396, shutdown)
 * and of java/src/main/native_knn (KNN initialize / load / findKnn).  A Java, Python or Go binding needs nothing else.
 *
 * All functions return 0 on success, a negative value on failure (dsstne_last_error() has the text) unless noted.
 * One context per process (runtime/DsstneContext.h:28-30).
 */
#ifndef DSSTNE_CAPI_H
#define DSSTNE_CAPI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct dsstne_context dsstne_context;

const char* dsstne_last_error(void);

/* Dsstne.load (Dsstne.cpp:136-143): GpuContext::Startup + LoadNeuralNetworkNetCDF + top-K result buffers of max_k x batch. */
dsstne_context* dsstne_load(const char* network_file, uint32_t batch, int max_k);

/* Same context, network given in memory instead of a file: a chain or DAG of fully connected layers.
 * layer_kind: NNLayer::Kind ordinals (0 input, 1 hidden, 2 output); layer_activation: Activation ordinals;
 * layer_sparse: 1 for sparse input layers.  Weight w connects weight_in[w] -> weight_out[w] (layer numbers), holds
 * weights[w] = [width(in)][width(out)] fp32 row-major and biases[w] = [width(out)]. */
dsstne_context* dsstne_create(const char* name, uint32_t batch, int max_k, uint32_t num_layers, const char* const* layer_names,
                              const uint32_t* layer_kind, const uint32_t* layer_width, const uint32_t* layer_activation,
                              const uint32_t* layer_sparse, const char* const* layer_dataset, uint32_t num_weights,
                              const uint32_t* weight_in, const uint32_t* weight_out, const float* const* weights,
                              const float* const* biases);

/* The training tool's start-up (utils/Train.cpp:119-133) up to the first prediction: LoadNetCDF(dataset_file), then
 * LoadNeuralNetworkJSON(definition_file, batch, datasets) (engine/NNNetwork.cpp:2792-3760: "N": "auto" layers are sized by
 * the data set they name), then LoadDataSets.  Weights start from each layer's "WeightInit" scheme and `seed`
 * (GpuContext::SetRandomSeed); the context owns the data sets.  NULL + dsstne_last_error() on failure. */
dsstne_context* dsstne_load_definition(const char* definition_file, const char* dataset_file, uint32_t batch, int max_k, uint64_t seed);

/* Weights and biases of the connection input_layer -> output_layer (NNWeight::GetWeights/GetBiases/SetWeights/SetBiases,
 * engine/NNWeight.cpp:938-1057): weights [width(in)][width(out)] fp32 row-major, biases [width(out)].  A NULL array is skipped. */
int dsstne_get_weights(dsstne_context* ctx, const char* input_layer, const char* output_layer, float* weights, size_t weight_count,
                       float* biases, size_t bias_count);
int dsstne_set_weights(dsstne_context* ctx, const char* input_layer, const char* output_layer, const float* weights, size_t weight_count,
                       const float* biases, size_t bias_count);

/* Dsstne.shutdown: deletes the network, the datasets created by dsstne_load_datasets and the device context. */
void dsstne_shutdown(dsstne_context* ctx);

/* NNNetwork::SaveNetCDF */
int dsstne_save_network(dsstne_context* ctx, const char* network_file);

/* Dsstne.load_datasets (Dsstne.cpp:155-191) -> DsstneContext::initInputLayerDataSets: one empty dataset per entry,
 * bound to the input layer of the same dataset name, followed by one priming prediction.
 * data_type: NNDataSetEnums::DataType, attributes: NNDataSetEnums::Attributes (0 dense or 1 sparse). */
int dsstne_load_datasets(dsstne_context* ctx, uint32_t count, const char* const* names, const uint32_t* data_type,
                         const uint32_t* attributes, const uint32_t* width, const uint32_t* examples, const float* sparse_density);

/* General dataset creation for the flavours the descriptor route cannot express (indexed, weighted, explicit capacity):
 * NNDataSet<T>(examples, uniqueExamples, sparseDataSize, dim, isIndexed, isWeighted, name) (engine/NNTypes.h:447-450).
 * boolean != 0 additionally marks the data as 0/1 (the attribute a NetCDF file would carry).  Binds like dsstne_load_datasets
 * once `last` != 0. */
int dsstne_add_sparse_dataset(dsstne_context* ctx, const char* name, uint32_t data_type, uint32_t width, uint32_t examples,
                              uint32_t unique_examples, uint64_t sparse_capacity, int indexed, int weighted, int boolean, int last);

/* NNDataSet<T>::LoadSparseData / LoadIndexedData / LoadDataWeight / LoadDenseData on dataset `name` (Dsstne.cpp:300-345). */
int dsstne_load_sparse_data(dsstne_context* ctx, const char* name, const uint64_t* sparse_start, const uint64_t* sparse_end,
                            const void* sparse_data, const uint32_t* sparse_index);
int dsstne_load_indexed_data(dsstne_context* ctx, const char* name, const uint32_t* index);
int dsstne_load_data_weight(dsstne_context* ctx, const char* name, const float* weight);
int dsstne_load_dense_data(dsstne_context* ctx, const char* name, const void* data);

/* NNNetwork::SetPosition + PredictBatch; results stay on the device. */
int dsstne_predict_batch(dsstne_context* ctx, uint32_t position);
/* kCalculateTopK on the output layer into the context's device buffers (Dsstne.cpp:372); filter_dataset != NULL applies
 * that sparse dataset as the per-sample filter inside the kernel (NNRecsGenerator semantics). */
int dsstne_topk(dsstne_context* ctx, const char* layer, uint32_t k, const char* filter_dataset);
/* Copies the last top-K results to the host: scores/indexes are [rows][k]. */
int dsstne_get_topk(dsstne_context* ctx, const char* layer, uint32_t rows, uint32_t k, float* scores, uint32_t* indexes);
/* No counterpart in the reference.  A network runs on two lanes by default: consecutive dsstne_predict_batch calls alternate
 * between two sets of unit and result buffers on two device streams, so a batch's kernels overlap with those of the batch
 * before it (NNNetwork::SetLanes).  dsstne_get_topk reads the batch predicted last; dsstne_get_topk_previous the one before
 * it, waiting for that batch only — a loop that issues batch i+1 and then collects batch i keeps the device busy.
 * dsstne_set_lanes(ctx, 1) goes back to one set of buffers and one stream; up to four lanes can be asked for (consecutive
 * batches then take turns on as many sets of buffers). */
int dsstne_get_topk_previous(dsstne_context* ctx, const char* layer, uint32_t rows, uint32_t k, float* scores, uint32_t* indexes);
int dsstne_set_lanes(dsstne_context* ctx, uint32_t lanes);
/* No counterpart in the reference (NNNetwork::SetDeferredOutput).  By default a wide output layer that feeds nothing else is
 * computed together with the dsstne_topk that follows dsstne_predict_batch, in one pass that never stores the layer's
 * [batch x width] result; dsstne_get_units / dsstne_get_unit_buffer compute it when asked.  defer == 0: every layer is stored
 * by dsstne_predict_batch, as in the reference. */
int dsstne_set_deferred_output(dsstne_context* ctx, int defer);
/* No counterpart in the reference (NNNetwork::SetSplitProducts).  split != 0: dense layers wide enough for the tiled kernel form
 * their fp32 products from bf16 matrix instructions (dsx_fc_forward_split in dsx.h): as close to the exact sums as fp32
 * multiplication, not bit-identical to it, about 1.5 times as fast; those layers' weights are kept a second time as bf16 planes.
 * Off by default. */
int dsstne_set_split_products(dsstne_context* ctx, int split);
/* Dsstne.predict in one call: position 0, predict, unfiltered (filter_dataset NULL) or filtered top-k, copy back. */
int dsstne_predict(dsstne_context* ctx, const char* layer, uint32_t k, const char* filter_dataset, float* scores, uint32_t* indexes);
/* NNLayer::GetUnits: the layer's [batch][width] activations. */
int dsstne_get_units(dsstne_context* ctx, const char* layer, float* units, size_t count);
/* NNNetwork::GetUnitBuffer (engine/NNNetwork.cpp:2006-2020): device address of the layer's [batch][stride] activations of the
 * batch predicted last, as the reference's JNI predict takes it (Dsstne.cpp:366).  The call returns once that batch's
 * forward pass has finished on the device, so the caller may read the memory with any copy or kernel of its own; the
 * address changes from batch to batch with more than one lane (fetch it per batch, as the reference's callers do).  NULL on failure. */
void* dsstne_get_unit_buffer(dsstne_context* ctx, const char* layer);
/* NNLayer::SetUnits (engine/NNLayer.cpp:318-368 group): overwrites the layer's unit buffer (batch x stride values) from the host. */
int dsstne_set_units(dsstne_context* ctx, const char* layer, const float* units, size_t count);
int dsstne_sync(void);
/* Event timing around calls on the library stream: milliseconds between start and stop. */
int dsstne_timer_start(void);
int dsstne_timer_stop(float* ms);

/* ---- KNN (java/src/main/native_knn/com_amazon_dsstne_knn_KNearestNeighborsCuda.cpp:185-262) ---- */
typedef struct dsstne_knn dsstne_knn;
dsstne_knn* dsstne_knn_create(uint32_t batch, uint32_t max_k);
/* The same with the item storage named like the JNI's dataType argument ("fp32" or "fp16": astdl::knn::getDataTypeFromString,
 * knn/KnnData.cpp:81-91; an unknown name fails). */
dsstne_knn* dsstne_knn_create_typed(uint32_t batch, uint32_t max_k, const char* data_type);
/* (data_type "fp32-split", which the reference does not have: fp32 storage with the inner products formed from bf16 matrix
 * instructions, dsx_knn_search_split in dsx.h) */
/* KnnData::load from rows in memory: items is [rows][dim] row-major; keys may be NULL (row numbers are used). */
int dsstne_knn_load(dsstne_knn* knn, const float* items, uint32_t rows, uint32_t dim, const char* const* keys);
/* KnnData::load from a text file "key<kv_delim>v0<vec_delim>v1..." */
int dsstne_knn_load_file(dsstne_knn* knn, const char* file, char kv_delim, char vec_delim);
/* KnnExactGpu::search: queries [size][dim]; scores [size][k]; keys come back as row numbers of the item table in `indexes`
 * (parsed from the string keys when they are numeric, else the load order). */
int dsstne_knn_search(dsstne_knn* knn, uint32_t k, const float* queries, uint32_t size, float* scores, uint32_t* indexes);
int dsstne_knn_elapsed(dsstne_knn* knn, float* gemm_ms, float* topk_ms);
void dsstne_knn_destroy(dsstne_knn* knn);

#ifdef __cplusplus
}
#endif
#endif
