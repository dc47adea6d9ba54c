// capi.cpp — C ABI over the C++ inference classes (include/dsstne_capi.h).
#include <cstring>
#include <cstdarg>
#include <stdexcept>

#include "amazon/dsstne/engine/NNTypes.h"
#include "amazon/dsstne/knn/KnnExactGpu.h"
#include "amazon/dsstne/runtime/DsstneContext.h"
#include "dsstne_capi.h"

using namespace std;

static thread_local char g_err[1024] = "";

static int fail(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return -1;
}

struct dsstne_context {
    DsstneContext* dc = nullptr;       // file-loaded networks
    NNNetwork* network = nullptr;      // in-memory networks (dc == nullptr)
    uint32_t batch = 0;
    int maxK = 0;
    map<string, NNDataSetBase*> datasets;
    vector<NNDataSetBase*> pending;
    map<string, GpuBuffer<NNFloat>*> scores[DSX_MAX_LANES];      // per lane of the network
    map<string, GpuBuffer<uint32_t>*> indexes[DSX_MAX_LANES];

    NNNetwork* net() const { return dc ? dc->getNetwork() : network; }
    GpuBuffer<NNFloat>* scoreBuf(const string& layer) { return dc ? dc->getOutputScoresBuffer(layer) : scores[network->GetLane()].at(layer); }
    GpuBuffer<uint32_t>* indexBuf(const string& layer) { return dc ? dc->getOutputIndexesBuffer(layer) : indexes[network->GetLane()].at(layer); }
};

#define CAPI_TRY try {
#define CAPI_CATCH(ret)                          \
    }                                            \
    catch (std::exception & e)                   \
    {                                            \
        fail("%s: %s", __func__, e.what());      \
        return ret;                              \
    }

template <typename T>
static NNDataSetBase* makeSparse(const char* name, uint32_t width, uint32_t examples, uint32_t unique, uint64_t cap, int indexed, int weighted)
{
    return new NNDataSet<T>(examples, unique, (size_t)cap, NNDataSetDimensions(width), indexed != 0, weighted != 0, name);
}

// Top-K result buffers of in-memory networks: one pair per output layer.
static void makeResultBuffers(dsstne_context* c)
{
    if (c->maxK <= 0) return;
    vector<const NNLayer*> outs;
    for (auto it = c->network->GetLayers(NNLayer::Kind::Output, outs); it != outs.end(); ++it) {
        for (int lane = 0; lane < DSX_MAX_LANES; lane++) {
            // (pinned host memory that the device writes straight into: a batch's results are batch x k pairs, and reading them
            // back is then a wait for the lane and a host copy, no transfer of its own)
            c->scores[lane][(*it)->GetName()] = new GpuBuffer<NNFloat>((size_t)c->maxK * c->batch, false, true);
            c->indexes[lane][(*it)->GetName()] = new GpuBuffer<uint32_t>((size_t)c->maxK * c->batch, false, true);
        }
    }
}

extern "C" {

const char* dsstne_last_error(void) { return g_err; }

dsstne_context* dsstne_load(const char* network_file, uint32_t batch, int max_k)
{
    CAPI_TRY
    dsstne_context* c = new dsstne_context();
    c->dc = new DsstneContext(network_file, batch, max_k);
    c->batch = batch;
    c->maxK = max_k;
    return c;
    CAPI_CATCH(nullptr)
}

dsstne_context* dsstne_create(const char* name, uint32_t batch, int max_k, uint32_t num_layers, const char* const* layer_names,
                              const uint32_t* layer_kind, const uint32_t* layer_width, const uint32_t* layer_activation,
                              const uint32_t* layer_sparse, const char* const* layer_dataset, uint32_t num_weights,
                              const uint32_t* weight_in, const uint32_t* weight_out, const float* const* weights,
                              const float* const* biases)
{
    CAPI_TRY
    static char arg0[] = "dsstne-capi";
    char* argv = arg0;
    getGpu().Startup(1, &argv);
    getGpu().SetRandomSeed(12134ULL);
    NNNetworkDescriptor nd;
    nd._name = name ? name : "network";
    nd._kind = NNNetwork::Kind::FeedForward;
    for (uint32_t i = 0; i < num_layers; i++) {
        NNLayerDescriptor ld;
        ld._name = layer_names[i];
        ld._kind = (NNLayer::Kind)layer_kind[i];
        ld._type = NNLayer::Type::FullyConnected;
        ld._Nx = layer_width[i];
        ld._dimensions = 1;
        ld._activation = (Activation)layer_activation[i];
        ld._attributes = (layer_sparse && layer_sparse[i]) ? NNLayer::Attributes::Sparse : NNLayer::Attributes::None;
        if (layer_dataset && layer_dataset[i]) ld._dataSet = layer_dataset[i];
        nd._vLayerDescriptor.push_back(ld);
    }
    for (uint32_t w = 0; w < num_weights; w++) {
        if (weight_in[w] >= num_layers || weight_out[w] >= num_layers) {
            fail("dsstne_create: weight %u connects unknown layers", w);
            return nullptr;
        }
        NNWeightDescriptor wd;
        wd._inputLayer = layer_names[weight_in[w]];
        wd._outputLayer = layer_names[weight_out[w]];
        wd._width = layer_width[weight_out[w]];
        wd._height = layer_width[weight_in[w]];
        const size_t n = (size_t)wd._width * wd._height;
        wd._vWeight.assign(weights[w], weights[w] + n);
        wd._vBias.assign(biases[w], biases[w] + wd._width);
        nd._vLayerDescriptor[weight_out[w]]._vSource.push_back(wd._inputLayer);
        nd._vWeightDescriptor.push_back(std::move(wd));
    }
    dsstne_context* c = new dsstne_context();
    c->network = CreateNeuralNetwork(nd, batch);
    getGpu().SetNeuralNetwork(c->network);
    c->batch = batch;
    c->maxK = max_k;
    makeResultBuffers(c);
    return c;
    CAPI_CATCH(nullptr)
}

dsstne_context* dsstne_load_definition(const char* definition_file, const char* dataset_file, uint32_t batch, int max_k, uint64_t seed)
{
    CAPI_TRY
    static char arg0[] = "dsstne-capi";
    char* argv = arg0;
    getGpu().Startup(1, &argv);
    getGpu().SetRandomSeed((unsigned long)seed);
    vector<NNDataSetBase*> vDataSet = LoadNetCDF(dataset_file);
    if (vDataSet.empty()) {
        fail("dsstne_load_definition: no data set could be read from %s", dataset_file);
        getGpu().Shutdown();
        return nullptr;
    }
    NNNetwork* network = LoadNeuralNetworkJSON(definition_file, batch, vDataSet);
    if (!network) {
        for (auto d : vDataSet) delete d;
        getGpu().Shutdown();
        fail("dsstne_load_definition: %s could not be loaded", definition_file);
        return nullptr;
    }
    dsstne_context* c = new dsstne_context();
    c->network = network;
    getGpu().SetNeuralNetwork(network);
    c->batch = batch;
    c->maxK = max_k;
    network->LoadDataSets(vDataSet);
    for (auto d : vDataSet) c->datasets[d->_name] = d;
    network->SetPosition(0);
    makeResultBuffers(c);
    return c;
    CAPI_CATCH(nullptr)
}

int dsstne_get_weights(dsstne_context* c, const char* input_layer, const char* output_layer, float* weights, size_t weight_count,
                       float* biases, size_t bias_count)
{
    CAPI_TRY
    NNWeight* w = c->net()->GetWeight(input_layer, output_layer);
    if (!w) return fail("dsstne_get_weights: no connection %s -> %s", input_layer, output_layer);
    if (weights) {
        vector<NNFloat> v;
        if (!w->GetWeights(v) || v.size() > weight_count) return fail("dsstne_get_weights: %zu weights do not fit %zu", v.size(), weight_count);
        std::copy(v.begin(), v.end(), weights);
    }
    if (biases) {
        vector<NNFloat> v;   // the getters only ever grow the vector they are given
        if (!w->GetBiases(v) || v.size() > bias_count) return fail("dsstne_get_weights: %zu biases do not fit %zu", v.size(), bias_count);
        std::copy(v.begin(), v.end(), biases);
    }
    return 0;
    CAPI_CATCH(-1)
}

int dsstne_set_weights(dsstne_context* c, const char* input_layer, const char* output_layer, const float* weights, size_t weight_count,
                       const float* biases, size_t bias_count)
{
    CAPI_TRY
    NNWeight* w = c->net()->GetWeight(input_layer, output_layer);
    if (!w) return fail("dsstne_set_weights: no connection %s -> %s", input_layer, output_layer);
    if (weights && !w->SetWeights(vector<NNFloat>(weights, weights + weight_count))) return fail("dsstne_set_weights: weights refused");
    if (biases && !w->SetBiases(vector<NNFloat>(biases, biases + bias_count))) return fail("dsstne_set_weights: biases refused");
    return 0;
    CAPI_CATCH(-1)
}

void dsstne_shutdown(dsstne_context* c)
{
    if (!c) return;
    for (int lane = 0; lane < DSX_MAX_LANES; lane++) {
        for (auto& kv : c->scores[lane]) delete kv.second;
        for (auto& kv : c->indexes[lane]) delete kv.second;
    }
    if (c->dc) {
        delete c->dc;   // deletes its network and datasets, shuts the device down
    } else {
        delete c->network;
        for (auto& kv : c->datasets) delete kv.second;
        getGpu().Shutdown();
    }
    delete c;
}

int dsstne_save_network(dsstne_context* c, const char* network_file)
{
    CAPI_TRY
    return c->net()->SaveNetCDF(network_file) ? 0 : fail("dsstne_save_network: failed");
    CAPI_CATCH(-1)
}

static int bindPending(dsstne_context* c)
{
    NNNetwork* network = c->net();
    network->LoadDataSets(c->pending);
    for (auto d : c->pending) c->datasets[d->_name] = d;
    c->pending.clear();
    network->PredictBatch();   // primes every buffer once (runtime/DsstneContext.cpp:111-123)
    network->SetPosition(0);
    return 0;
}

int dsstne_load_datasets(dsstne_context* c, uint32_t count, const char* const* names, const uint32_t* data_type, const uint32_t* attributes,
                         const uint32_t* width, const uint32_t* examples, const float* sparse_density)
{
    CAPI_TRY
    for (uint32_t i = 0; i < count; i++) {
        NNDataSetDescriptor d;
        d._name = names[i];
        d._dataType = (NNDataSetEnums::DataType)data_type[i];
        d._attributes = attributes[i];
        d._dim = NNDataSetDimensions(width[i]);
        d._examples = examples[i];
        d._sparseDensity = sparse_density[i];
        c->pending.push_back(createNNDataSet(d));
    }
    return bindPending(c);
    CAPI_CATCH(-1)
}

int dsstne_add_sparse_dataset(dsstne_context* c, const char* name, uint32_t data_type, uint32_t width, uint32_t examples,
                              uint32_t unique_examples, uint64_t sparse_capacity, int indexed, int weighted, int boolean, int last)
{
    CAPI_TRY
    NNDataSetBase* d = nullptr;
    switch (data_type) {
    case NNDataSetEnums::UInt: d = makeSparse<uint32_t>(name, width, examples, unique_examples, sparse_capacity, indexed, weighted); break;
    case NNDataSetEnums::Int: d = makeSparse<int32_t>(name, width, examples, unique_examples, sparse_capacity, indexed, weighted); break;
    case NNDataSetEnums::LLInt: d = makeSparse<int64_t>(name, width, examples, unique_examples, sparse_capacity, indexed, weighted); break;
    case NNDataSetEnums::ULLInt: d = makeSparse<uint64_t>(name, width, examples, unique_examples, sparse_capacity, indexed, weighted); break;
    case NNDataSetEnums::Float: d = makeSparse<float>(name, width, examples, unique_examples, sparse_capacity, indexed, weighted); break;
    case NNDataSetEnums::Double: d = makeSparse<double>(name, width, examples, unique_examples, sparse_capacity, indexed, weighted); break;
    case NNDataSetEnums::UChar: d = makeSparse<unsigned char>(name, width, examples, unique_examples, sparse_capacity, indexed, weighted); break;
    case NNDataSetEnums::Char: d = makeSparse<char>(name, width, examples, unique_examples, sparse_capacity, indexed, weighted); break;
    default: return fail("dsstne_add_sparse_dataset: unsupported data type %u", data_type);
    }
    if (boolean) d->_attributes |= NNDataSetEnums::Boolean;
    c->pending.push_back(d);
    // a dataset that matches no layer (a filter) is only registered
    if (last) return bindPending(c);
    return 0;
    CAPI_CATCH(-1)
}

static NNDataSetBase* findDataSet(dsstne_context* c, const char* name)
{
    auto it = c->datasets.find(name);
    if (it != c->datasets.end()) return it->second;
    for (auto d : c->pending)
        if (d->_name == name) return d;
    // datasets created through a file-loaded context live on the layers
    vector<const NNLayer*> ins;
    for (auto l = c->net()->GetLayers(NNLayer::Kind::Input, ins); l != ins.end(); ++l)
        if ((*l)->GetDataSet() && (*l)->GetDataSet()->_name == name) return (*l)->GetDataSet();
    throw std::runtime_error(string("unknown dataset ") + name);
}

int dsstne_load_sparse_data(dsstne_context* c, const char* name, const uint64_t* sparse_start, const uint64_t* sparse_end,
                            const void* sparse_data, const uint32_t* sparse_index)
{
    CAPI_TRY
    NNDataSetBase* d = findDataSet(c, name);
    // a Boolean dataset has no value array and its kernels read none: nothing is copied or uploaded for it.  Any other set
    // without values gets zeros of the right length.
    vector<uint8_t> zeros;
    if (!sparse_data && !(d->_attributes & NNDataSetEnums::Boolean)) {
        zeros.assign((size_t)sparse_end[d->_uniqueExamples - 1] * 8, 0);
        sparse_data = zeros.data();
    }
    d->LoadSparseData(sparse_start, sparse_end, sparse_data, sparse_index);
    return 0;
    CAPI_CATCH(-1)
}

int dsstne_load_indexed_data(dsstne_context* c, const char* name, const uint32_t* index)
{
    CAPI_TRY
    findDataSet(c, name)->LoadIndexedData(index);
    return 0;
    CAPI_CATCH(-1)
}

int dsstne_load_data_weight(dsstne_context* c, const char* name, const float* weight)
{
    CAPI_TRY
    findDataSet(c, name)->LoadDataWeight(weight);
    return 0;
    CAPI_CATCH(-1)
}

int dsstne_load_dense_data(dsstne_context* c, const char* name, const void* data)
{
    CAPI_TRY
    findDataSet(c, name)->LoadDenseData(data);
    return 0;
    CAPI_CATCH(-1)
}

int dsstne_predict_batch(dsstne_context* c, uint32_t position)
{
    CAPI_TRY
    NNNetwork* n = c->net();
    if (position != n->GetPosition()) n->SetPosition(position);
    n->PredictBatch();
    return 0;
    CAPI_CATCH(-1)
}

int dsstne_topk(dsstne_context* c, const char* layer, uint32_t k, const char* filter_dataset)
{
    CAPI_TRY
    if ((int)k > c->maxK) return fail("dsstne_topk: k = %u is > maxK = %d", k, c->maxK);
    NNNetwork* n = c->net();
    if (filter_dataset)
        n->CalculateFilteredTopK(layer, k, findDataSet(c, filter_dataset), c->scoreBuf(layer), c->indexBuf(layer));
    else {
        // like the JNI path, which calls the raw kernel: k up to 256 (NNNetwork::CalculateTopK stops at 128)
        n->CalculateFilteredTopK(layer, k, NULL, NULL, NULL, NULL, c->scoreBuf(layer)->_pDevData, c->indexBuf(layer)->_pDevData);
    }
    return 0;
    CAPI_CATCH(-1)
}

int dsstne_get_topk(dsstne_context* c, const char* layer, uint32_t rows, uint32_t k, float* scores, uint32_t* indexes)
{
    CAPI_TRY
    GpuBuffer<NNFloat>* s = c->scoreBuf(layer);
    GpuBuffer<uint32_t>* i = c->indexBuf(layer);
    if (s->_bManaged && i->_bManaged) {   // the kernels wrote into host memory: wait for the batch's lane, then it is all there
        dsxFatal(dsx_sync_lane(c->net()->GetLane()), "dsstne_get_topk");
        memcpy(scores, s->_pSysData, (size_t)rows * k * sizeof(float));
        memcpy(indexes, i->_pSysData, (size_t)rows * k * sizeof(uint32_t));
        return 0;
    }
    dsxFatal(dsx_memcpy_d2h_pair(scores, s->_pDevData, (size_t)rows * k * sizeof(float), indexes, i->_pDevData,
                                 (size_t)rows * k * sizeof(uint32_t)),
             "dsstne_get_topk");
    return 0;
    CAPI_CATCH(-1)
}

int dsstne_get_topk_previous(dsstne_context* c, const char* layer, uint32_t rows, uint32_t k, float* scores, uint32_t* indexes)
{
    CAPI_TRY
    NNNetwork* n = c->net();
    if (n->GetLanes() < 2) return fail("dsstne_get_topk_previous: the network runs on one lane");
    const int lane = (int)((n->GetLane() + n->GetLanes() - 1) % n->GetLanes());
    GpuBuffer<NNFloat>* s = c->dc ? c->dc->getOutputScoresBuffer(layer, lane) : c->scores[lane].at(layer);
    GpuBuffer<uint32_t>* i = c->dc ? c->dc->getOutputIndexesBuffer(layer, lane) : c->indexes[lane].at(layer);
    if (s->_bManaged && i->_bManaged) {
        dsxFatal(dsx_sync_lane(lane), "dsstne_get_topk_previous");
        memcpy(scores, s->_pSysData, (size_t)rows * k * sizeof(float));
        memcpy(indexes, i->_pSysData, (size_t)rows * k * sizeof(uint32_t));
        return 0;
    }
    dsxFatal(dsx_memcpy_d2h_lane(lane, scores, s->_pDevData, (size_t)rows * k * sizeof(float)), "dsstne_get_topk_previous");
    dsxFatal(dsx_memcpy_d2h_lane(lane, indexes, i->_pDevData, (size_t)rows * k * sizeof(uint32_t)), "dsstne_get_topk_previous");
    return 0;
    CAPI_CATCH(-1)
}

int dsstne_set_lanes(dsstne_context* c, uint32_t lanes)
{
    CAPI_TRY
    return c->net()->SetLanes(lanes) ? 0 : fail("dsstne_set_lanes: %u lanes (1..%d)", lanes, DSX_MAX_LANES);
    CAPI_CATCH(-1)
}

int dsstne_set_split_products(dsstne_context* c, int split)
{
    CAPI_TRY
    return c->net()->SetSplitProducts(split != 0) ? 0 : fail("dsstne_set_split_products failed");
    CAPI_CATCH(-1)
}

int dsstne_set_deferred_output(dsstne_context* c, int defer)
{
    CAPI_TRY
    return c->net()->SetDeferredOutput(defer != 0) ? 0 : fail("dsstne_set_deferred_output failed");
    CAPI_CATCH(-1)
}

int dsstne_predict(dsstne_context* c, const char* layer, uint32_t k, const char* filter_dataset, float* scores, uint32_t* indexes)
{
    int rc = dsstne_predict_batch(c, 0);
    if (rc) return rc;
    rc = dsstne_topk(c, layer, k, filter_dataset);
    if (rc) return rc;
    NNNetwork* n = c->net();
    return dsstne_get_topk(c, layer, std::min<uint32_t>(n->GetBatch(), n->GetExamples()), k, scores, indexes);
}

int dsstne_get_units(dsstne_context* c, const char* layer, float* units, size_t count)
{
    CAPI_TRY
    NNLayer* l = c->net()->GetLayer(layer);
    if (!l) return fail("dsstne_get_units: unknown layer %s", layer);
    NNFloat* p = c->net()->GetUnitBuffer(layer);
    if (!p) return fail("dsstne_get_units: layer %s has no unit buffer", layer);
    if (count > c->net()->GetBufferSize(layer)) return fail("dsstne_get_units: %zu values requested, the layer holds %zu", count, (size_t)c->net()->GetBufferSize(layer));
    dsxFatal(dsx_memcpy_d2h(units, p, count * sizeof(float)), "dsstne_get_units");
    return 0;
    CAPI_CATCH(-1)
}

void* dsstne_get_unit_buffer(dsstne_context* c, const char* layer)
{
    CAPI_TRY
    NNFloat* p = c->net()->GetUnitBuffer(layer);
    if (!p) fail("dsstne_get_unit_buffer: layer %s is unknown or has no unit buffer", layer);
    return (void*)p;
    CAPI_CATCH(NULL)
}

int dsstne_set_units(dsstne_context* c, const char* layer, const float* units, size_t count)
{
    CAPI_TRY
    NNLayer* l = c->net()->GetLayer(layer);
    if (!l) return fail("dsstne_set_units: unknown layer %s", layer);
    std::vector<NNFloat> v(units, units + count);
    if (!const_cast<NNLayer*>(l)->SetUnits(v)) return fail("dsstne_set_units: layer %s refused %zu values", layer, count);
    return 0;
    CAPI_CATCH(-1)
}

int dsstne_sync(void) { return dsx_sync(); }
int dsstne_timer_start(void) { return dsx_timer_start(); }
int dsstne_timer_stop(float* ms) { return dsx_timer_stop(ms); }

// ------------------------------------------------------------------------------------------------------------------- KNN

struct dsstne_knn {
    astdl::knn::KnnData* data = nullptr;
    astdl::knn::KnnExactGpu* knn = nullptr;
    bool numericKeys = true;
};

dsstne_knn* dsstne_knn_create(uint32_t batch, uint32_t max_k) { return dsstne_knn_create_typed(batch, max_k, "fp32"); }

dsstne_knn* dsstne_knn_create_typed(uint32_t batch, uint32_t max_k, const char* data_type)
{
    CAPI_TRY
    dsstne_knn* k = new dsstne_knn();
    k->data = new astdl::knn::KnnData(1, (int)batch, (int)max_k, astdl::knn::getDataTypeFromString(data_type ? data_type : "fp32"));
    k->knn = new astdl::knn::KnnExactGpu(k->data);
    return k;
    CAPI_CATCH(nullptr)
}

int dsstne_knn_load(dsstne_knn* k, const float* items, uint32_t rows, uint32_t dim, const char* const* keys)
{
    CAPI_TRY
    vector<string> skeys;
    if (keys)
        for (uint32_t i = 0; i < rows; i++) skeys.push_back(keys[i]);
    ArrayDataReader reader(items, rows, (int)dim, keys ? skeys.data() : nullptr);
    k->data->load(0, &reader);
    k->numericKeys = (keys == nullptr);
    return 0;
    CAPI_CATCH(-1)
}

int dsstne_knn_load_file(dsstne_knn* k, const char* file, char kv_delim, char vec_delim)
{
    CAPI_TRY
    std::map<int, std::string> files = {{0, file}};
    k->data->load(files, kv_delim, vec_delim);
    k->numericKeys = false;
    return 0;
    CAPI_CATCH(-1)
}

int dsstne_knn_search(dsstne_knn* k, uint32_t kk, const float* queries, uint32_t size, float* scores, uint32_t* indexes)
{
    CAPI_TRY
    vector<string> keys((size_t)size * kk);
    k->knn->search((int)kk, queries, (int)size, keys.data(), scores);
    if (indexes) {
        if (k->numericKeys) {
            for (size_t i = 0; i < keys.size(); i++) indexes[i] = keys[i].empty() ? 0xffffffffu : (uint32_t)stoul(keys[i]);
        } else {
            // keys are arbitrary labels: report their load order
            std::map<string, uint32_t> order;
            const auto& all = k->data->hKeys[0];
            for (uint32_t i = 0; i < all.size(); i++) order.emplace(all[i], i);
            for (size_t i = 0; i < keys.size(); i++) {
                auto it = order.find(keys[i]);
                indexes[i] = it == order.end() ? 0xffffffffu : it->second;
            }
        }
    }
    return 0;
    CAPI_CATCH(-1)
}

int dsstne_knn_elapsed(dsstne_knn* k, float* gemm_ms, float* topk_ms)
{
    if (gemm_ms) *gemm_ms = k->data->elapsedSgemm[0];
    if (topk_ms) *topk_ms = k->data->elapsedTopK[0];
    return 0;
}

void dsstne_knn_destroy(dsstne_knn* k)
{
    if (!k) return;
    delete k->knn;
    delete k->data;
    delete k;
}

}  // extern "C"
